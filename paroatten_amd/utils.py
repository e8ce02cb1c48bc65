"""The reference's `paroattention.utils` (paroattention/utils.py:4-34): the earlier form of the step-end
callback.  It differs from the one in prefetch_utils in two points that are kept here: the step is not
wrapped round the number of scheduler steps, and the transformer receives the NORMALISED step
(step + 1) / total as a float while the attn1 processors receive the mask-timestep index."""
from __future__ import annotations

import torch

from .prefetch_utils import _CallbackBase


class TimestepCallback(_CallbackBase):
    def __init__(self, num_timestep_for_sparse_mask=10):
        super().__init__()
        self.timestep_history = []
        self.num_timestep_for_sparse_mask = num_timestep_for_sparse_mask

    def on_step_end(self, pipeline, step, timestep, callback_kwargs):
        self.timestep_history.append({
            "step": step,
            "timestep": timestep.item() if torch.is_tensor(timestep) else timestep,
            "latents": callback_kwargs.get("latents", None),
        })
        total_steps = len(pipeline.scheduler.timesteps)
        normalized_timestep = (step + 1) / total_steps
        sparse_mask_timestep = int(normalized_timestep * self.num_timestep_for_sparse_mask)
        transformer = pipeline.transformer
        transformer.i_timestep = normalized_timestep
        blocks = getattr(transformer, "transformer_blocks", None)
        if blocks is None:
            blocks = transformer.blocks
        for block in blocks:
            block.attn1.processor.i_timestep = sparse_mask_timestep
        return callback_kwargs

    def callback_fn(self, pipeline, step_index, timestep, callback_kwargs):
        return self.on_step_end(pipeline, step_index, timestep, callback_kwargs)
