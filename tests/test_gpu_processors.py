"""GPU tests of the callers around the kernels: mask bit packing, the mask prefetch stream, and the
CogVideoX / Wan attention processors driven with a stand-in attention module (diffusers is not
installed; the processors only use `to_q/to_k/to_v/norm_q/norm_k/to_out/heads`)."""
import numpy as np
import pytest
import torch

from conftest import cosine
from oracle import paro_oracle as O
from paroatten_amd import synth

pytestmark = pytest.mark.gpu


class _Attn(torch.nn.Module):
    def __init__(self, heads, head_dim, norm, seed):
        super().__init__()
        torch.manual_seed(seed)
        dim = heads * head_dim
        self.heads = heads
        self.to_q = torch.nn.Linear(dim, dim)
        self.to_k = torch.nn.Linear(dim, dim)
        self.to_v = torch.nn.Linear(dim, dim)
        self.to_out = torch.nn.ModuleList([torch.nn.Linear(dim, dim), torch.nn.Dropout(0.0)])
        if norm == "layer":      # CogVideoX: LayerNorm over the head dimension, after the head split
            self.norm_q, self.norm_k = torch.nn.LayerNorm(head_dim), torch.nn.LayerNorm(head_dim)
        elif norm == "rms":      # Wan: RMS norm across heads, before the head split
            self.norm_q, self.norm_k = torch.nn.RMSNorm(dim), torch.nn.RMSNorm(dim)
        else:
            self.norm_q = self.norm_k = None
        self.is_cross_attention = False
        self.add_k_proj = None


def _rel_rms(a, b):
    return ((a.float() - b.float()).pow(2).mean().sqrt() / b.float().pow(2).mean().sqrt()).item()


@pytest.mark.parametrize("n", [16, 1000, 48 * 30 * 30 + 5])
def test_mask_pack_unpack_kernels(dev, n):
    from paroatten_amd import _lib
    lib = _lib.load()
    g = torch.Generator().manual_seed(n)
    m = torch.rand(n, generator=g) < 0.3
    nbytes = lib.paro_mask_bits_bytes(n)
    assert nbytes == (n + 7) // 8
    md = m.to(dev)
    bits = torch.zeros((nbytes + 15) // 16 * 16, dtype=torch.uint8, device=dev)
    _lib.check(lib.paro_mask_pack(_lib.ptr(md), _lib.ptr(bits), n, _lib.stream_of(md)))
    want = np.packbits(m.numpy(), bitorder="little")
    assert np.array_equal(bits.cpu().numpy()[:nbytes], want)
    back = torch.full((n,), 7, dtype=torch.uint8, device=dev)
    _lib.check(lib.paro_mask_unpack(_lib.ptr(bits), _lib.ptr(back), n, _lib.stream_of(md)))
    assert torch.equal(back.cpu().bool(), m) and int(back.max()) <= 1


def test_prefetch_stream_serves_the_right_mask(dev):
    """in-order use, a timestep change at the layer wrap (a misprediction), a jump, a timestep past
    the last mask timestep (the callback's final value) and reuse after reset()."""
    from paroatten_amd.prefetch_utils import SparseMaskPrefetchStream
    T, L, H, nb = 3, 4, 2, 37
    g = torch.Generator().manual_seed(0)
    masks = torch.rand(T, L, H, nb, nb, generator=g) < 0.4
    ps = SparseMaskPrefetchStream(masks, device=dev)
    assert (ps.n_timestep, ps.n_transformer_block, ps.n_head, ps.mask_len, ps.num_iterations) == (T, L, H, nb, T * L)
    assert ps.double_buffer[0].shape == (H, nb, nb) and ps.double_buffer[0].dtype == torch.bool
    seq = [(0, b) for b in range(L)] + [(0, b) for b in range(L)] + [(1, b) for b in range(L)]
    seq += [(2, 3), (0, 1), (3, 0), (3, 1)]
    sink = torch.zeros(H, nb, nb, dtype=torch.int32, device=dev)
    for i, (t, b) in enumerate(seq):
        m = ps.mask_for(t, b)
        sink += m            # a queued reader of the buffer, as the attention kernel is
        assert torch.equal(m.cpu(), masks[min(t, T - 1), b]), (i, t, b)
    assert ps.i_iter == len(seq)
    ps.reset()
    assert ps.i_iter == 0
    assert torch.equal(ps.mask_for(0, 0).cpu(), masks[0, 0])
    want = sum(masks[min(t, T - 1), b].int() for t, b in seq)
    assert torch.equal(sink.cpu(), want)


def _cog_case(dev, dtype=torch.bfloat16, seed=0):
    H, D, grid, n_text, B = 2, 64, (4, 8, 12), 32, 2
    n_img = grid[0] * grid[1] * grid[2]
    N = n_text + n_img
    attn = _Attn(H, D, "layer", seed).to(dev, dtype)
    g = torch.Generator().manual_seed(seed + 1)
    hidden = torch.randn(B, n_img, H * D, generator=g).to(dev, dtype)
    text = torch.randn(B, n_text, H * D, generator=g).to(dev, dtype)
    from paroatten_amd import rope
    cos, sin = rope.rope_table_cog(D, grid)
    nb = (N + 63) // 64
    T, L = 2, 3
    masks = torch.stack([torch.stack([synth.make_block_mask(H, nb, 0.5, seed=10 + t * L + l) for l in range(L)])
                         for t in range(T)])
    plan = synth.make_permute_plan(L, H, seed=seed + 2)
    return attn, hidden, text, (cos, sin), masks, plan, grid, n_text


def _cog_expected(attn, hidden, text, rotary, mask, plan, i_block, grid, n_text, smooth_k=False):
    """The reference's sequence (cogvideox.py:139-235) with the oracle in place of the kernels."""
    hs = torch.cat([text, hidden], dim=1)
    B, N, _ = hs.shape
    H = attn.heads
    q = attn.norm_q(attn.to_q(hs).view(B, N, H, -1).transpose(1, 2))
    k = attn.norm_k(attn.to_k(hs).view(B, N, H, -1).transpose(1, 2))
    v = attn.to_v(hs).view(B, N, H, -1).transpose(1, 2)
    o = O.paro_path(q.cpu().contiguous(), k.cpu().contiguous(), v.cpu().contiguous(), mask[None].expand(B, -1, -1, -1), plan, i_block,
                    grid, n_text, rotary[0], rotary[1], smooth_k=smooth_k)
    o = o.to(hs.device).transpose(1, 2).reshape(B, N, -1).to(hs.dtype)
    o = attn.to_out[1](attn.to_out[0](o))
    return o[:, n_text:], o[:, :n_text], q, k, v


@torch.no_grad()
@pytest.mark.parametrize("smooth_k", [False, True])
def test_cogvideox_processor_against_oracle(dev, smooth_k):
    from paroatten_amd import PARO_CogVideoXAttnProcessor2_0
    attn, hidden, text, rotary, masks, plan, grid, n_text = _cog_case(dev)
    proc = PARO_CogVideoXAttnProcessor2_0(grid=grid, smooth_k=smooth_k)
    proc.permute_plan, proc.i_block, proc.i_timestep = plan, 1, 1
    proc.sparse_mask = masks.to(dev)
    out_h, out_t = proc(attn, hidden, text, image_rotary_emb=(rotary[0].to(dev), rotary[1].to(dev)))
    ref_h, ref_t, *_ = _cog_expected(attn, hidden, text, rotary, masks[1, 1], plan, 1, grid, n_text, smooth_k)
    assert out_h.shape == hidden.shape and out_t.shape == text.shape and out_h.dtype == hidden.dtype
    for got, ref in ((out_h, ref_h), (out_t, ref_t)):
        assert cosine(got.cpu(), ref.cpu()) >= 0.999
        assert _rel_rms(got, ref) <= 0.05          # FP8 P and V: 3.7..4.1 % of the attention output
    stats = proc.get_time_stats()
    assert stats["total_ms"] > 0 and proc.call_count == 1


@torch.no_grad()
def test_cogvideox_processor_accuracy_mode(dev):
    """pv_f16=True: the processor's attention runs the float16 P.V product; against the oracle the attention's
    share of the error drops from FP8's 4 % to what the bfloat16 projections round to."""
    from paroatten_amd import PARO_CogVideoXAttnProcessor2_0
    attn, hidden, text, rotary, masks, plan, grid, n_text = _cog_case(dev)
    ref_h, ref_t, *_ = _cog_expected(attn, hidden, text, rotary, masks[1, 1], plan, 1, grid, n_text, True)
    rms = {}
    for pv16 in (False, True):
        proc = PARO_CogVideoXAttnProcessor2_0(grid=grid, smooth_k=True, pv_f16=pv16)
        proc.permute_plan, proc.i_block, proc.i_timestep = plan, 1, 1
        proc.sparse_mask = masks.to(dev)
        out_h, out_t = proc(attn, hidden, text, image_rotary_emb=(rotary[0].to(dev), rotary[1].to(dev)))
        rms[pv16] = max(_rel_rms(out_h, ref_h), _rel_rms(out_t, ref_t))
        assert cosine(out_h.cpu(), ref_h.cpu()) >= (0.9999 if pv16 else 0.999)
    assert rms[True] <= 0.012, rms           # bfloat16 rounding of the attention output and of the projection
    assert rms[True] < 0.5 * rms[False], rms


@torch.no_grad()
def test_cogvideox_processor_prefetch_equals_resident_mask(dev):
    from paroatten_amd import PARO_CogVideoXAttnProcessor2_0
    from paroatten_amd.prefetch_utils import SparseMaskPrefetchStream
    attn, hidden, text, rotary, masks, plan, grid, n_text = _cog_case(dev, seed=5)
    rot = (rotary[0].to(dev), rotary[1].to(dev))
    a = PARO_CogVideoXAttnProcessor2_0(grid=grid)
    b = PARO_CogVideoXAttnProcessor2_0(grid=grid)
    a.permute_plan = b.permute_plan = plan
    a.sparse_mask = masks.to(dev)
    b.prefetch_stream = SparseMaskPrefetchStream(masks, device=dev)
    for t, l in ((0, 0), (0, 1), (0, 2), (1, 0), (1, 1)):
        a.i_timestep = b.i_timestep = t
        a.i_block = b.i_block = l
        ra = a(attn, hidden, text, image_rotary_emb=rot)
        rb = b(attn, hidden, text, image_rotary_emb=rot)
        assert torch.equal(ra[0], rb[0]) and torch.equal(ra[1], rb[1])


@torch.no_grad()
def test_cogvideox_processor_dense_fallback(dev):
    """i_timestep < 0: dense attention (cogvideox.py:215-221) == SDPA on the rotated projections."""
    from paroatten_amd import PARO_CogVideoXAttnProcessor2_0
    attn, hidden, text, rotary, masks, plan, grid, n_text = _cog_case(dev, seed=9)
    proc = PARO_CogVideoXAttnProcessor2_0(grid=grid)
    proc.permute_plan, proc.i_block, proc.i_timestep = plan, 0, -1
    out_h, out_t = proc(attn, hidden, text, image_rotary_emb=(rotary[0].to(dev), rotary[1].to(dev)))
    hs = torch.cat([text, hidden], dim=1)
    B, N, _ = hs.shape
    q = attn.norm_q(attn.to_q(hs).view(B, N, attn.heads, -1).transpose(1, 2)).cpu()
    k = attn.norm_k(attn.to_k(hs).view(B, N, attn.heads, -1).transpose(1, 2)).cpu()
    v = attn.to_v(hs).view(B, N, attn.heads, -1).transpose(1, 2)
    q[:, :, n_text:] = O.rope_apply_cog(q[:, :, n_text:], rotary[0], rotary[1])
    k[:, :, n_text:] = O.rope_apply_cog(k[:, :, n_text:], rotary[0], rotary[1])
    o = torch.nn.functional.scaled_dot_product_attention(q.to(dev), k.to(dev), v)
    o = attn.to_out[0](o.transpose(1, 2).reshape(B, N, -1))
    assert torch.allclose(out_h.float(), o[:, n_text:].float(), atol=2e-2, rtol=2e-2)
    assert torch.allclose(out_t.float(), o[:, :n_text].float(), atol=2e-2, rtol=2e-2)


@torch.no_grad()
def test_wan_processor_against_oracle(dev):
    from paroatten_amd import PARO_WanAttnProcessor2_0
    H, D, grid, B = 2, 128, (3, 6, 16), 1
    N = grid[0] * grid[1] * grid[2]
    dtype = torch.bfloat16
    attn = _Attn(H, D, "rms", seed=21).to(dev, dtype)
    g = torch.Generator().manual_seed(22)
    hidden = torch.randn(B, N, H * D, generator=g).to(dev, dtype)
    freqs = O.rope_table_wan(D, grid)                      # complex128 [1,1,N,D/2], as WanRotaryPosEmbed returns
    nb = (N + 63) // 64
    masks = torch.stack([torch.stack([synth.make_block_mask(H, nb, 0.6, seed=30 + l) for l in range(2)])])
    plan = synth.make_permute_plan(2, H, seed=23)
    proc = PARO_WanAttnProcessor2_0(grid=grid)
    proc.permute_plan, proc.i_block, proc.i_timestep = plan, 1, 0
    proc.sparse_mask = masks.to(dev)
    out = proc(attn, hidden, rotary_emb=freqs.to(dev))
    assert out.shape == hidden.shape and out.dtype == dtype

    q = attn.norm_q(attn.to_q(hidden)).unflatten(2, (H, -1)).transpose(1, 2).cpu()
    k = attn.norm_k(attn.to_k(hidden)).unflatten(2, (H, -1)).transpose(1, 2).cpu()
    v = attn.to_v(hidden).unflatten(2, (H, -1)).transpose(1, 2).cpu()
    q, k = O.rope_apply_wan(q, freqs), O.rope_apply_wan(k, freqs)
    o = O.paro_path(q.contiguous(), k.contiguous(), v.contiguous(), masks[0, 1][None], plan, 1, grid, 0, smooth_k=False)
    ref = attn.to_out[0](o.to(dev).transpose(1, 2).flatten(2, 3).to(dtype))
    assert cosine(out.cpu(), ref.cpu()) >= 0.999
    assert _rel_rms(out, ref) <= 0.05

    # later diffusers versions pass (cos, sin) as real tensors [1, N, 1, D], every pair's frequency repeated over
    # the pair: the same tables, hence the same bits
    fr = freqs.reshape(N, D // 2)
    pair = (fr.real.float().repeat_interleave(2, dim=1).view(1, N, 1, D).to(dev),
            fr.imag.float().repeat_interleave(2, dim=1).view(1, N, 1, D).to(dev))
    assert torch.equal(proc(attn, hidden, rotary_emb=pair), out)

    # cross-attention inputs (another key length) take the dense path
    ctx = torch.randn(B, 40, H * D, generator=g).to(dev, dtype)
    out_x = proc(attn, hidden, encoder_hidden_states=ctx)
    qx = attn.norm_q(attn.to_q(hidden)).unflatten(2, (H, -1)).transpose(1, 2)
    kx = attn.norm_k(attn.to_k(ctx)).unflatten(2, (H, -1)).transpose(1, 2)
    vx = attn.to_v(ctx).unflatten(2, (H, -1)).transpose(1, 2)
    ox = torch.nn.functional.scaled_dot_product_attention(qx, kx, vx).transpose(1, 2).flatten(2, 3)
    assert torch.allclose(out_x.float(), attn.to_out[0](ox).float(), atol=2e-2, rtol=2e-2)


def test_processor_rejects_unknown_grid(dev):
    from paroatten_amd import PARO_CogVideoXAttnProcessor2_0
    attn, hidden, text, rotary, masks, plan, grid, n_text = _cog_case(dev)
    proc = PARO_CogVideoXAttnProcessor2_0()          # no grid given and 384 image tokens are not CogVideoX's
    proc.permute_plan, proc.i_block, proc.i_timestep = plan, 0, 0
    proc.sparse_mask = masks.to(dev)
    with pytest.raises(ValueError):
        proc(attn, hidden, text)


@torch.no_grad()
def test_pipeline_wiring_over_layers_and_steps(dev):
    """set_paro_processors + TimestepCallback on a stand-in transformer: three blocks, five denoising
    steps mapped onto two mask timesteps; the prefetch-stream run equals the resident-mask run in every
    block and step, and the mask timestep follows the callback's arithmetic."""
    import types

    from paroatten_amd import wan
    from paroatten_amd.prefetch_utils import SparseMaskPrefetchStream, TimestepCallback, mask_timestep_index
    H, D, grid, n_text, B, L, T, steps = 2, 64, (2, 4, 8), 0, 1, 3, 2, 5
    N = grid[0] * grid[1] * grid[2]
    nb = (N + 63) // 64
    masks = torch.stack([torch.stack([synth.make_block_mask(H, nb, 0.7, seed=50 + t * L + l, band=0) for l in range(L)])
                         for t in range(T)])
    plan = synth.make_permute_plan(L, H, seed=51)

    def make_transformer():
        blocks = [types.SimpleNamespace(attn1=_Attn(H, D, "rms", seed=60 + i).to(dev, torch.bfloat16)) for i in range(L)]
        for b in blocks:
            b.attn1.processor = None
        return types.SimpleNamespace(blocks=blocks)

    ta, tb = make_transformer(), make_transformer()
    pa = wan.set_paro_processors(ta, plan, sparse_mask=masks.to(dev), grid=grid)
    stream = SparseMaskPrefetchStream(masks, device=dev)
    pb = wan.set_paro_processors(tb, plan, prefetch_stream=stream, grid=grid)
    assert [p.i_block for p in pa] == [0, 1, 2] and all(p.i_timestep == 0 for p in pb)
    assert all(isinstance(p, wan.PARO_WanAttnProcessor2_0) for p in pa)
    with pytest.raises(ValueError):
        wan.set_paro_processors(ta, plan)
    cb_a, cb_b = TimestepCallback(T), TimestepCallback(T)
    sched = types.SimpleNamespace(timesteps=list(range(steps)))
    pipe_a = types.SimpleNamespace(transformer=ta, scheduler=sched)
    pipe_b = types.SimpleNamespace(transformer=tb, scheduler=sched)
    g = torch.Generator().manual_seed(52)
    x = torch.randn(B, N, H * D, generator=g).to(dev, torch.bfloat16)
    freqs = O.rope_table_wan(D, grid).to(dev)
    seen = []
    for step in range(steps):
        ha = hb = x
        for l in range(L):
            ha = ta.blocks[l].attn1.processor(ta.blocks[l].attn1, ha, rotary_emb=freqs)
            hb = tb.blocks[l].attn1.processor(tb.blocks[l].attn1, hb, rotary_emb=freqs)
            assert torch.equal(ha, hb), (step, l)
        seen.append(pa[0].i_timestep)
        cb_a.on_step_end(pipe_a, step, torch.tensor(float(step)), {})
        cb_b.on_step_end(pipe_b, step, torch.tensor(float(step)), {})
    want = [0] + [min(mask_timestep_index(s, steps, T), T) for s in range(steps - 1)]
    assert seen == want and ta.i_timestep == mask_timestep_index(steps - 1, steps, T)
    assert stream.i_iter == steps * L
    assert sum(p.call_count for p in pb) == steps * L and pb[0].get_time_stats()["total_ms"] > 0
