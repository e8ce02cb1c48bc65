"""The two forms of the attention kernel at head size 64 — one wave per 64-row q-block (the default without
lse) and two waves per q-block (flag PARO_ATTN_TWO_WAVES) — compute the same arithmetic in a different
order of issue: their outputs must agree bit for bit, on every path through the loop (one, two, odd and
even numbers of kept blocks per row, rows without any, tails, causal diagonals, grouped heads, strided
layouts, the fast path's second pass after an overflow, the inverse permutation folded into the stores)."""
import pytest
import torch

from conftest import assert_attention_close
from oracle import paro_oracle as O
from paroatten_amd import synth

pytestmark = pytest.mark.gpu


def _both(dev, q, k, v, mask, **kw):
    import paroatten_amd as P
    a = P.paroattn_qk_int8_pv_fp16_cuda(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), **kw)
    b = P.paroattn_qk_int8_pv_fp16_cuda(q.to(dev), k.to(dev), v.to(dev), mask.to(dev), two_waves=True, **kw)
    torch.cuda.synchronize()
    return a.cpu(), b.cpu()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("exact", [False, True])
@pytest.mark.parametrize("causal", [False, True])
def test_kept_block_counts_and_tails(dev, dtype, exact, causal):
    """Row i of head 0 keeps min(i, nb) blocks starting at the diagonal (0, 1, 2, 3 ... kept blocks, so the
    loop runs zero, one, an odd and an even number of times and both ring stages end a row); head 1 keeps
    random blocks; head 2 everything.  N is not a multiple of 64, so the last block has dead columns."""
    B, H, N, D = 2, 3, 64 * 11 - 21, 64
    nb = (N + 63) // 64
    q, k, v = synth.make_qkv(B, H, N, D, dtype, seed=3)
    mask = torch.zeros(H, nb, nb, dtype=torch.bool)
    for i in range(nb):
        for j in range(i):
            mask[0, i, (i - j) % nb if causal else (i + j) % nb] = True
    mask[1] = synth.make_block_mask(1, nb, 0.35, seed=9)[0]
    mask[2] = True
    a, b = _both(dev, q, k, v, mask, is_causal=causal, exact_exp=exact, smooth_k=True)
    assert torch.isfinite(a.float()).all()
    assert torch.equal(a, b)
    assert torch.count_nonzero(a[:, 0, :64]) == 0          # the row of head 0 without a kept block
    # and the shared result is the oracle's
    km = k.float().mean(dim=2, keepdim=True).to(dtype)
    q8, qs, k8, ks = O.per_warp_int8(q, k, km=km, BLKQ=64, WARPQ=32, BLKK=64)
    o_ref, _ = O.sparse_attention(q8, k8, v, qs, ks, mask[None].expand(B, H, nb, nb), D ** -0.5, is_causal=causal,
                                  out_dtype=torch.float32)
    a_ref, _ = O.sparse_attention(q8, k8, v.abs(), qs, ks, mask[None].expand(B, H, nb, nb), D ** -0.5,
                                  is_causal=causal, out_dtype=torch.float32)
    assert_attention_close(a, o_ref, a_ref)


def test_grouped_heads_and_token_major_layout(dev):
    B, H, Hkv, N, D = 1, 4, 2, 700, 64
    q, _, _ = synth.make_qkv(B, H, N, D, torch.float16, seed=21)
    _, k, v = synth.make_qkv(B, Hkv, N, D, torch.float16, seed=22)
    nb = (N + 63) // 64
    mask = synth.make_block_mask(H, nb, 0.5, seed=23)
    a, b = _both(dev, q, k, v, mask)
    assert torch.equal(a, b)
    # [B,N,H,D]: rows of one head are H*D bytes apart in K8, which the tile mover has to follow
    qn, kn, vn = (t.transpose(1, 2).contiguous() for t in (q, k, v))
    an, bn = _both(dev, qn, kn, vn, mask, tensor_layout="NHD")
    assert torch.equal(an, bn)
    assert torch.equal(an.transpose(1, 2), a)


@pytest.mark.parametrize("causal", [False, True])
def test_second_pass_after_overflow(dev, causal):
    """Scores that climb by three nats per key block force the fast path to refresh the maximum and build the
    weights of a block a second time, in block after block and in both halves of the q-block."""
    from test_gpu_attention import _ramp_case
    B, H, N, D = 1, 2, 1024 - 19, 64
    nb = (N + 63) // 64
    for pattern in ("ramp", "spike"):
        q, k, v = _ramp_case(B, H, N, D, torch.float16, 71, pattern)
        for mask in (torch.ones(H, nb, nb, dtype=torch.bool), synth.make_block_mask(H, nb, 0.5, seed=5)):
            a, b = _both(dev, q, k, v, mask, is_causal=causal, smooth_k=False)
            assert torch.isfinite(a.float()).all()
            assert torch.equal(a, b)


def test_folded_inverse_permutation(dev):
    """paro_attn_sparse_unpermute_fwd stores q-row r at its un-permuted token: same bytes from both forms."""
    from paroatten_amd import _qattn_sm80 as qattn, permute as PM, quant as Q
    B, H, D, grid, n_text = 1, 6, 64, (3, 5, 7), 23
    N = n_text + grid[0] * grid[1] * grid[2]
    nb = (N + 63) // 64
    q, k, v = (t.to(dev) for t in synth.make_qkv(B, H, N, D, torch.bfloat16, seed=31))
    orders = torch.arange(6, dtype=torch.int32, device=dev)
    mask = synth.make_block_mask(H, nb, 0.6, seed=32).to(dev)
    q8, qs, k8, ks = Q.per_warp_int8(q, k, None, BLKQ=64, WARPQ=32, BLKK=64)
    v8, vsc, vm = Q.per_channel_fp8(v)
    outs = []
    for two in (False, True):
        o = torch.zeros(B, N, H, D, dtype=torch.bfloat16, device=dev).transpose(1, 2)   # token-major buffer, HND view
        qattn.attn_sparse_prepacked(q8, k8, v8, vsc, vm, o, qs, ks, D ** -0.5, mask, unpermute=(orders, grid, n_text),
                                    two_waves=two)
        outs.append(o.cpu())
    assert torch.equal(outs[0], outs[1])
    assert float(outs[0].float().abs().max()) > 0
