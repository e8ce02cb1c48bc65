"""Sparse-mask staging: the reference's `paroattention.prefetch_utils`
(paroattention/prefetch_utils.py:4-59; the Wan twin paroattention/prefetch_wan.py:4-56).

`TimestepCallback` keeps the reference's arithmetic.  `SparseMaskPrefetchStream` keeps its fields
and its purpose (the [T,L,H,nb,nb] plan stays on the host, two [H,nb,nb] device buffers alternate,
the copy of the next layer's mask overlaps the attention of this one) with three changes:
  * the host copy is bit-packed in pinned memory (8x smaller; Wan 720p: 8.9 GB -> 1.1 GB) and
    unpacked on the device by paro_mask_unpack on the copy stream;
  * buffers carry the index of the mask they hold and completion events, so a consumer never reads
    a buffer whose copy is in flight and a copy never overwrites a buffer a queued kernel reads;
  * the mask is addressed by (i_timestep, i_block) rather than by a call counter, so runs with
    more denoising steps than mask timesteps, or a counter that was not reset, still get the right
    mask (a wrong prediction costs one synchronous copy, never a wrong mask).
"""
from __future__ import annotations

import numpy as np
import torch

from . import _lib
from ._lib import load, ptr

try:  # diffusers is optional: the callback only needs its calling convention
    from diffusers.callbacks import PipelineCallback as _CallbackBase
except Exception:  # pragma: no cover - depends on the environment
    class _CallbackBase:
        def __init__(self, cutoff_step_ratio=1.0, cutoff_step_index=None):
            self.config = {"cutoff_step_ratio": cutoff_step_ratio, "cutoff_step_index": cutoff_step_index}

        @property
        def tensor_inputs(self):
            return []


def mask_timestep_index(step: int, total_steps: int, num_timestep_for_sparse_mask: int) -> int:
    """Mask timestep for the step AFTER `step` (the callback runs at step end):
    int(((step % total) + 1) / total * T)  (prefetch_utils.py:22-25)."""
    step = step % total_steps
    return int((step + 1) / total_steps * num_timestep_for_sparse_mask)


class TimestepCallback(_CallbackBase):
    """Pipeline callback that writes the sparse-mask timestep into the transformer and every attn1
    processor (CogVideoX: `transformer_blocks`, Wan: `blocks`)."""

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
        self.sparse_mask_timestep = mask_timestep_index(step, total_steps, self.num_timestep_for_sparse_mask)
        transformer = pipeline.transformer
        transformer.i_timestep = self.sparse_mask_timestep
        blocks = getattr(transformer, "transformer_blocks", None)
        if blocks is None:
            blocks = transformer.blocks
        for block in blocks:
            block.attn1.processor.i_timestep = self.sparse_mask_timestep
        return callback_kwargs

    # diffusers' PipelineCallback.__call__ dispatches to callback_fn
    def callback_fn(self, pipeline, step_index, timestep, callback_kwargs):
        return self.on_step_end(pipeline, step_index, timestep, callback_kwargs)


def pack_mask_bits(mask: torch.Tensor) -> torch.Tensor:
    """Host side of paro_mask_pack: bool [..., n] -> uint8 [..., ceil(n/8) rounded up to 16 bytes],
    bit i of byte j = element 8j+i.  Rows are padded to 16 bytes so that every row of a pinned
    [iterations, row] array can be copied to an aligned device buffer."""
    m = mask.reshape(mask.shape[0], -1).numpy()
    bits = np.packbits(m, axis=1, bitorder="little")
    row = (bits.shape[1] + 15) // 16 * 16
    out = torch.zeros((bits.shape[0], row), dtype=torch.uint8)
    out[:, :bits.shape[1]] = torch.from_numpy(bits)
    return out


class SparseMaskPrefetchStream:
    def __init__(self, sparse_mask: torch.Tensor, device=None, batch_size: int = 2):
        """sparse_mask: bool [T, L, H, nb, nb] on the CPU."""
        if sparse_mask.dim() != 5 or sparse_mask.shape[-1] != sparse_mask.shape[-2]:
            raise ValueError(f"sparse_mask must be [T,L,H,nb,nb], got {tuple(sparse_mask.shape)}")
        if sparse_mask.is_cuda:
            raise ValueError("sparse_mask must live on the CPU (it is staged to the device per layer)")
        load()
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        self.n_timestep, self.n_transformer_block, self.n_head, self.mask_len, _ = sparse_mask.shape
        self.num_iterations = self.n_timestep * self.n_transformer_block
        self.mask_elems = self.n_head * self.mask_len * self.mask_len
        packed = pack_mask_bits(sparse_mask.bool().reshape(self.num_iterations, self.mask_elems))
        # pinned and packed; `sparse_mask` keeps the reference's field name for the host copy
        self.sparse_mask = torch.empty(packed.shape, dtype=torch.uint8, pin_memory=True)
        self.sparse_mask.copy_(packed)
        self.i_iter = 0
        self.batch_size = batch_size
        shape = [self.n_head, self.mask_len, self.mask_len]
        self.double_buffer = [torch.empty(shape, dtype=torch.bool, device=self.device) for _ in range(2)]
        self._bits = [torch.empty(packed.shape[1], dtype=torch.uint8, device=self.device) for _ in range(2)]
        self._last = 0
        self._held = [-1, -1]                      # flat mask index each buffer holds (or is being filled with)
        self._ready = [torch.cuda.Event(), torch.cuda.Event()]
        self.stream = torch.cuda.Stream(device=self.device)   # default priority
        self._stage(0, 0, after=None)
        self.stream.synchronize()

    def reset(self):
        """Call after each pipeline run (prefetch_utils.py:57-59)."""
        self.i_iter = 0

    def flat_index(self, i_timestep: int, i_block: int) -> int:
        t = min(max(int(i_timestep), 0), self.n_timestep - 1)   # the callback's last step maps to T
        return t * self.n_transformer_block + int(i_block)

    def _stage(self, index: int, buf: int, after):
        """Queue on the copy stream: wait `after` (an event on the consumer's stream), H2D of the
        packed mask, unpack into double_buffer[buf], record the buffer's ready event."""
        with torch.cuda.stream(self.stream):
            if after is not None:
                self.stream.wait_event(after)
            self._bits[buf].copy_(self.sparse_mask[index], non_blocking=True)
            _lib.on(self._bits[buf]).paro_mask_unpack(ptr(self._bits[buf]), ptr(self.double_buffer[buf]), self.mask_elems,
                                          _lib.stream_of(self._bits[buf]))
            self._ready[buf].record(self.stream)
        self._held[buf] = index

    def mask_for(self, i_timestep: int, i_block: int) -> torch.Tensor:
        """Device mask bool [H,nb,nb] of (i_timestep, i_block), valid on the caller's current
        stream; queues the copy of the next block's mask behind the work already queued there."""
        index = self.flat_index(i_timestep, i_block)
        main = torch.cuda.current_stream(self.device)
        if index in self._held:
            buf = self._held.index(index)
        else:                                       # not predicted: stage now, behind queued readers
            buf = 1 - self._last
            fence = torch.cuda.Event()
            fence.record(main)
            self._stage(index, buf, after=fence)
        main.wait_event(self._ready[buf])
        self._last = buf
        # prediction: the next block of this timestep; after the last block, block 0 of the same
        # timestep (the callback moves to the next mask timestep only every few denoising steps)
        t = index // self.n_transformer_block
        nxt = index + 1 if (index + 1) % self.n_transformer_block else t * self.n_transformer_block
        if nxt != index and nxt not in self._held:
            # the other buffer was last read by kernels already queued on `main`
            fence = torch.cuda.Event()
            fence.record(main)
            self._stage(nxt, 1 - buf, after=fence)
        self.i_iter += 1
        return self.double_buffer[buf]
