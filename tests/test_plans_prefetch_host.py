"""Host-side logic around the path (no GPU): plan file formats, mask expansion for the kernel, the
timestep callback's arithmetic, bit packing of masks."""
import types

import numpy as np
import pytest
import torch

from paroatten_amd import plans, prefetch_utils


def test_plan_files_round_trip(tmp_path):
    p_path, s_path = plans.write_synthetic_plans(tmp_path, T=2, L=3, H=4, nb_img=10, density=0.4, seed=3)
    pp = plans.load_permute_plan(p_path)
    sp = plans.load_sparse_plan(s_path)
    assert pp["permute"].shape == (3, 4) and pp["permute"].dtype == torch.int64
    assert int(pp["permute"].min()) >= 0 and int(pp["permute"].max()) <= 5
    assert pp["empty"].shape == (3, 4) and pp["empty"].dtype == torch.bool
    assert sp["sparse"].shape == (2, 3, 4, 10, 10) and sp["sparse"].dtype == torch.bool
    # exact block count per head, diagonal kept
    assert torch.all(sp["sparse"].sum(dim=(-1, -2)) == max(40, int((torch.arange(10)[:, None] - torch.arange(10)).abs().le(2).sum())))
    assert torch.all(torch.diagonal(sp["sparse"], dim1=-2, dim2=-1))
    assert torch.allclose(sp["dense_rate"], sp["sparse"].float().mean(dim=(-1, -2)))


def test_plan_validation():
    with pytest.raises(ValueError):
        plans.check_permute_plan({"permute": torch.tensor([[0, 6]])})
    with pytest.raises(ValueError):
        plans.check_permute_plan({"perm": torch.zeros(1, 1)})
    ok = plans.check_permute_plan({"permute": torch.tensor([[0, 5]], dtype=torch.int32)})
    assert ok["empty"].shape == (1, 2) and not ok["empty"].any()


def test_cog_kernel_mask_text_blocks():
    """pipeline_cogvideox.py:80,99-100: 4 leading rows/columns of ones, last row/column True;
    the image part is untouched elsewhere."""
    g = torch.Generator().manual_seed(0)
    s = torch.rand(2, 1, 3, 274, 274, generator=g) < 0.2
    m = plans.cog_kernel_mask(s)
    assert m.shape == (2, 1, 3, 278, 278)
    assert m[..., :4, :].all() and m[..., :, :4].all()
    assert m[..., -1, :].all() and m[..., :, -1].all()
    assert torch.equal(m[..., 4:-1, 4:-1], s[..., :-1, :-1])
    w = plans.wan_kernel_mask(s)
    assert w.shape == s.shape and w[..., -1, :].all() and w[..., :, -1].all()
    assert torch.equal(w[..., :-1, :-1], s[..., :-1, :-1])
    assert not s[..., -1, :].all()   # the input was not modified


@pytest.mark.parametrize("step,total,T,expect", [
    (0, 50, 10, 0), (3, 50, 10, 0), (4, 50, 10, 1), (48, 50, 10, 9), (49, 50, 10, 10),
    (50, 50, 10, 0), (0, 4, 4, 1), (2, 4, 4, 3), (7, 8, 4, 4),
])
def test_mask_timestep_index(step, total, T, expect):
    """prefetch_utils.py:22-25, worked by hand: int(((step % total)+1)/total*T)."""
    assert prefetch_utils.mask_timestep_index(step, total, T) == expect


@pytest.mark.parametrize("blocks_attr", ["transformer_blocks", "blocks"])
def test_timestep_callback_writes_every_processor(blocks_attr):
    procs = [types.SimpleNamespace(i_timestep=-5) for _ in range(3)]
    blocks = [types.SimpleNamespace(attn1=types.SimpleNamespace(processor=p)) for p in procs]
    transformer = types.SimpleNamespace(**{blocks_attr: blocks})
    pipe = types.SimpleNamespace(transformer=transformer, scheduler=types.SimpleNamespace(timesteps=list(range(20))))
    cb = prefetch_utils.TimestepCallback(num_timestep_for_sparse_mask=10)
    kw = {"latents": None}
    assert cb.on_step_end(pipe, 5, torch.tensor(801.0), kw) is kw
    assert transformer.i_timestep == 3 and all(p.i_timestep == 3 for p in procs)
    assert cb.timestep_history[0]["step"] == 5 and cb.timestep_history[0]["timestep"] == 801.0


def test_utils_timestep_callback_keeps_its_own_convention():
    """paroattention/utils.py:13-34: the transformer gets (step + 1) / total as a float, the processors the
    index int(that * T); worked by hand for step 5 of 20, T = 10: 0.3 and 3; step 25 is not wrapped: 1.3, 13"""
    from paroatten_amd import utils
    procs = [types.SimpleNamespace(i_timestep=-5) for _ in range(2)]
    blocks = [types.SimpleNamespace(attn1=types.SimpleNamespace(processor=p)) for p in procs]
    transformer = types.SimpleNamespace(transformer_blocks=blocks)
    pipe = types.SimpleNamespace(transformer=transformer, scheduler=types.SimpleNamespace(timesteps=list(range(20))))
    cb = utils.TimestepCallback(num_timestep_for_sparse_mask=10)
    kw = {"latents": None}
    assert cb.on_step_end(pipe, 5, 801, kw) is kw
    assert transformer.i_timestep == pytest.approx(0.3) and all(p.i_timestep == 3 for p in procs)
    cb.on_step_end(pipe, 25, 1, kw)
    assert transformer.i_timestep == pytest.approx(1.3) and all(p.i_timestep == 13 for p in procs)
    assert [h["step"] for h in cb.timestep_history] == [5, 25]


@pytest.mark.parametrize("n", [1, 7, 8, 9, 127, 128, 1000])
def test_pack_mask_bits_matches_numpy(n):
    g = torch.Generator().manual_seed(n)
    m = torch.rand(3, n, generator=g) < 0.5
    bits = prefetch_utils.pack_mask_bits(m)
    assert bits.shape[1] % 16 == 0 and bits.shape[1] >= (n + 7) // 8
    back = np.unpackbits(bits.numpy(), axis=1, bitorder="little")[:, :n]
    assert np.array_equal(back.astype(bool), m.numpy())
    # element 8j+i is bit i of byte j
    j, i = (n - 1) // 8, (n - 1) % 8
    assert bool((int(bits[0, j]) >> i) & 1) == bool(m[0, n - 1])


def test_processor_grid_and_table_cache_rules():
    """a token count does not fix (F,H,W): the explicit grid wins, a guessed one warns once; the
    rotary-table cache is keyed on the identity and version of the source tensors, not on an address"""
    from paroatten_amd.cogvideox import PARO_CogVideoXAttnProcessor2_0
    from paroatten_amd.wan import WAN_GRIDS, PARO_WanAttnProcessor2_0
    p = PARO_WanAttnProcessor2_0(grid=(21, 52, 30))
    assert p._grid_for(21 * 30 * 52, WAN_GRIDS) == (21, 52, 30)            # portrait: as given
    q = PARO_WanAttnProcessor2_0()
    with pytest.warns(UserWarning, match="assuming"):
        assert q._grid_for(21 * 30 * 52, WAN_GRIDS) == (21, 30, 52)
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        assert q._grid_for(21 * 30 * 52, WAN_GRIDS) == (21, 30, 52)        # only once
    with pytest.raises(ValueError):
        PARO_WanAttnProcessor2_0(grid=(21, 30, 52))._grid_for(100, WAN_GRIDS)
    c = PARO_CogVideoXAttnProcessor2_0()
    cos, sin = torch.zeros(8, 4, dtype=torch.float64), torch.ones(8, 4, dtype=torch.float64)   # converted: a copy
    a1 = c._tables((cos, sin), "cpu")
    assert c._tables((cos, sin), "cpu")[0] is a1[0]                        # same objects, unmodified: cached
    cos.add_(1.0)                                                          # modified in place: rebuilt
    a2 = c._tables((cos, sin), "cpu")
    assert a2[0] is not a1[0] and torch.equal(a2[0], cos.float())
    cos2 = cos.clone()                                                     # another object: rebuilt
    assert c._tables((cos2, sin), "cpu")[0] is not a2[0]
    # the processors of a model share ONE conversion per source (Wan hands every layer the same rotary tensor)
    from paroatten_amd.cogvideox import SHARED_TABLES
    c2 = PARO_CogVideoXAttnProcessor2_0()
    assert c2._tables((cos2, sin), "cpu")[0] is c._tables((cos2, sin), "cpu")[0]
    freqs = torch.polar(torch.ones(1, 1, 6, 4, dtype=torch.float64), torch.rand(1, 1, 6, 4, dtype=torch.float64))
    w1, w2 = PARO_WanAttnProcessor2_0(), PARO_WanAttnProcessor2_0()
    t1 = w1._tables(freqs, "cpu", 8)
    assert w2._tables(freqs, "cpu", 8)[0] is t1[0] and t1[0].shape == (6, 8)
    assert len(SHARED_TABLES._entries) <= SHARED_TABLES.KEEP                # bounded: the two most recent sources
    del freqs                                                               # the source is held weakly
    import gc
    gc.collect()
    assert any(r() is None for _, refs, _, _ in SHARED_TABLES._entries for r, _ in refs)
