"""The plan files as the example pipeline handles them (example/pipeline_cogvideox.py:72-136), end to
end on the GPU: write_synthetic_plans -> load_permute_plan / load_sparse_plan (weights-only loader) ->
cog_kernel_mask (4 text blocks of ones in front, last row and column forced) -> resident mask or
SparseMaskPrefetchStream -> PARO_CogVideoXAttnProcessor2_0 -> oracle, over mask timesteps x blocks,
including an out-of-order (mispredicted) block and the callback's final i_timestep == T."""
import pytest
import torch

from conftest import cosine
from oracle import paro_oracle as O
from paroatten_amd import plans, synth
from test_gpu_processors import _Attn, _cog_expected, _rel_rms

pytestmark = pytest.mark.gpu


def _setup(dev, tmp_path, H, grid, n_text, T, L, density, seed):
    from paroatten_amd import rope
    D = 64
    n_img = grid[0] * grid[1] * grid[2]
    N = n_text + n_img
    nb = (N + 63) // 64
    nb_img = nb - 4       # 226 text + the first 30 image tokens are 4 blocks (pipeline_cogvideox.py:80)
    p_path, s_path = plans.write_synthetic_plans(tmp_path, T=T, L=L, H=H, nb_img=nb_img, density=density, seed=seed)
    plan = plans.load_permute_plan(p_path)
    sparse = plans.load_sparse_plan(s_path)["sparse"]
    assert sparse.shape == (T, L, H, nb_img, nb_img)
    masks = plans.cog_kernel_mask(sparse)
    assert masks.shape == (T, L, H, nb, nb)
    attn = _Attn(H, D, "layer", seed).to(dev, torch.bfloat16)
    g = torch.Generator().manual_seed(seed + 1)
    hidden = torch.randn(1, n_img, H * D, generator=g).to(dev, torch.bfloat16)
    text = torch.randn(1, n_text, H * D, generator=g).to(dev, torch.bfloat16)
    return attn, hidden, text, rope.rope_table_cog(D, grid), masks, plan


@torch.no_grad()
def test_plan_files_to_processor_small(dev, tmp_path):
    """226 text tokens + a 3x10x15 grid (11 blocks, 7 of them image-only), 3 heads, 2 mask timesteps x 3
    blocks: every (timestep, block), visited out of order, through the resident mask and through the
    prefetch stream, against the oracle."""
    from paroatten_amd import PARO_CogVideoXAttnProcessor2_0
    from paroatten_amd.prefetch_utils import SparseMaskPrefetchStream
    grid, n_text, T, L = (3, 10, 15), 226, 2, 3
    attn, hidden, text, rotary, masks, plan = _setup(dev, tmp_path, 3, grid, n_text, T, L, 0.5, seed=70)
    rot = (rotary[0].to(dev), rotary[1].to(dev))
    a = PARO_CogVideoXAttnProcessor2_0(grid=grid)
    b = PARO_CogVideoXAttnProcessor2_0(grid=grid)
    a.permute_plan = b.permute_plan = plan
    a.sparse_mask = masks.to(dev)
    b.prefetch_stream = SparseMaskPrefetchStream(masks, device=dev, batch_size=1)
    # in order, then a jump back (not what the stream predicted), then the callback's final value T
    visits = [(0, 0), (0, 1), (0, 2), (1, 0), (1, 2), (1, 1), (0, 2), (T, 0)]
    for t, l in visits:
        a.i_timestep = b.i_timestep = t
        a.i_block = b.i_block = l
        ra = a(attn, hidden, text, image_rotary_emb=rot)
        rb = b(attn, hidden, text, image_rotary_emb=rot)
        assert torch.equal(ra[0], rb[0]) and torch.equal(ra[1], rb[1]), (t, l)
        ref_h, ref_t, *_ = _cog_expected(attn, hidden, text, rotary, masks[min(t, T - 1), l], plan, l, grid, n_text)
        for got, ref in ((ra[0], ref_h), (ra[1], ref_t)):
            assert cosine(got.cpu(), ref.cpu()) >= 0.999, (t, l)
            assert _rel_rms(got, ref) <= 0.05, (t, l)
    # the text blocks and the forced last row / column reached the kernel: with them cleared, the result differs
    a.i_timestep = b.i_timestep = 0
    a.i_block = b.i_block = 0
    intact = b(attn, hidden, text, image_rotary_emb=rot)[0]
    broken = masks.clone()
    broken[..., :4] = False
    a.sparse_mask = broken.to(dev)
    assert not torch.equal(a(attn, hidden, text, image_rotary_emb=rot)[0], intact)


@torch.no_grad()
def test_plan_files_to_processor_cogvideox_block_counts(dev, tmp_path):
    """the real CogVideoX token count (226 + 13x30x45 = 17776 tokens, 278 blocks, plan masks 274x274),
    two heads: one (timestep, block) against the oracle, the others resident == prefetched."""
    from paroatten_amd import PARO_CogVideoXAttnProcessor2_0
    from paroatten_amd.prefetch_utils import SparseMaskPrefetchStream
    wl = synth.WORKLOADS["cogvideox5b"]
    T, L = 2, 3
    attn, hidden, text, rotary, masks, plan = _setup(dev, tmp_path, 2, wl.grid, wl.n_text, T, L, 0.3, seed=80)
    assert masks.shape[-1] == wl.nb == 278
    rot = (rotary[0].to(dev), rotary[1].to(dev))
    a = PARO_CogVideoXAttnProcessor2_0()       # grid recognised from the token count (warns once)
    b = PARO_CogVideoXAttnProcessor2_0(grid=wl.grid)
    a.permute_plan = b.permute_plan = plan
    a.sparse_mask = masks.to(dev)
    b.prefetch_stream = SparseMaskPrefetchStream(masks, device=dev, batch_size=1)
    with pytest.warns(UserWarning, match="assuming"):
        for t in range(T):
            for l in range(L):
                a.i_timestep = b.i_timestep = t
                a.i_block = b.i_block = l
                ra = a(attn, hidden, text, image_rotary_emb=rot)
                rb = b(attn, hidden, text, image_rotary_emb=rot)
                assert torch.equal(ra[0], rb[0]) and torch.equal(ra[1], rb[1]), (t, l)
    ref_h, ref_t, *_ = _cog_expected(attn, hidden, text, rotary, masks[T - 1, L - 1], plan, L - 1, wl.grid, wl.n_text)
    for got, ref in ((ra[0], ref_h), (ra[1], ref_t)):
        assert cosine(got.cpu(), ref.cpu()) >= 0.999
        assert _rel_rms(got, ref) <= 0.05
