"""The per-layer sequence under HIP graph capture: rotated K mean -> one-pass preparation -> block-sparse
attention storing through the inverse permutation, captured once with torch.cuda.CUDAGraph and replayed
several times with eager work and synchronisations in between.  Every replay must reproduce the eager
result bit for bit: the library allocates nothing, synchronises nothing and keeps no state between calls
(the paced launch clears its counters with a small kernel, not a memset node), which is what makes it
capturable."""
import pytest
import torch

from paroatten_amd import synth

pytestmark = pytest.mark.gpu


def _sequence(dev, B, H, D, grid, n_text, dtype, density, pacing, seed):
    from paroatten_amd import _qattn_sm80 as qattn
    from paroatten_amd import permute as PM
    from paroatten_amd import rope
    N = n_text + grid[0] * grid[1] * grid[2]
    nb = (N + 63) // 64
    q, k, v = synth.make_qkv_device(B, H, N, D, dtype, seed=seed, device=dev)
    mask = synth.make_block_mask(H, nb, density, seed=seed + 1, device=dev)
    orders = PM.head_orders(synth.make_permute_plan(1, H, seed=seed + 2), 0, dev)
    cos, sin = (t.to(dev) for t in rope.rope_table_cog(D, grid))
    out = torch.zeros((B, N, H, D), dtype=dtype, device=dev)

    def run():
        km = PM.rope_k_mean(k, grid, n_text, cos, sin)
        ops = PM.rope_permute_quant(q, k, v, orders, grid, n_text, cos, sin, km=km)
        qattn.attn_sparse_prepacked(ops.q8, ops.k8, ops.v8, ops.v_scale, ops.v_mean, out.transpose(1, 2), ops.q_scale,
                                    ops.k_scale, D ** -0.5, mask, unpermute=(orders, grid, n_text), pacing=pacing)
    return run, out, (q, k, v)


@pytest.mark.parametrize("D,dtype,pacing", [(64, torch.float16, None), (128, torch.bfloat16, True)])
def test_sequence_replays_bit_identically(dev, D, dtype, pacing):
    # 2 x 12 heads of 32 + 8*16*24 = 3104 tokens (49 blocks): 1176 q-blocks, 147 per XCD, which with pacing
    # forced is more than the 128 workgroups resident on an XCD at D = 128, so the generation counters are in use
    run, out, (q, k, v) = _sequence(dev, 2, 12, D, (8, 16, 24), 32, dtype, 0.4, pacing, seed=5)
    run()                                   # eager: also resolves per-device addresses outside the capture
    torch.cuda.synchronize()
    want = out.clone()
    assert torch.isfinite(want.float()).all() and float(want.float().abs().max()) > 0

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):           # warm-up on the capture stream, as torch asks for
        run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for i in range(4):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), f"replay {i}"
        # the program's own eager work between replays: another launch of the same kernels on other data
        other, other_out, _ = _sequence(dev, 1, 3, D, (4, 6, 8), 0, dtype, 0.5, pacing, seed=50 + i)
        other()
        torch.cuda.synchronize()
        assert torch.isfinite(other_out.float()).all()

    # new inputs in the captured buffers: the replay computes on what the buffers hold now
    q2, k2, v2 = synth.make_qkv_device(*q.shape, dtype, seed=99, device=dev)
    q.copy_(q2); k.copy_(k2); v.copy_(v2)
    run()
    torch.cuda.synchronize()
    want2 = out.clone()
    assert not torch.equal(want2, want)
    out.fill_(float("nan"))
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), want2.view(torch.int16))
