"""The compiled PyTorch-ROCm C++ extension (paroatten_amd/_ext.so, csrc/torch_binding.cpp) against the
ctypes mirrors: both bind the same C ABI, so every result is compared bit for bit.  The extension's
submodules carry the reference's module names and positional signatures
(csrc/qattn/pybind_sm80.cpp:21-27, csrc/fused/pybind.cpp:21-33, csrc/rope/pybind.cpp:5-8)."""
import pytest
import torch

from paroatten_amd import synth


@pytest.fixture(scope="module")
def ext():
    import paroatten_amd
    try:
        return paroatten_amd.compiled_extension()
    except ImportError as e:     # not built, or torch's HIP libraries cannot be loaded in this process
        pytest.skip(f"compiled extension unavailable: {e} (build it with `python paroatten_amd/build.py`)")


def test_extension_imports_and_rejects_cpu_tensors(ext):
    x = torch.zeros(1, 1, 64, 64, dtype=torch.float16)
    o = torch.zeros(1, 1, 64, 64, dtype=torch.int8)
    s = torch.zeros(1, 1, 2)
    m = torch.ones(1, 1, 1, 1, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="Tensor input must be on CUDA"):
        ext._fused.quant_per_warp_int8_cuda(x, o, s, 64, 32, 1)
    with pytest.raises(RuntimeError, match="Tensor query must be on CUDA"):
        ext._qattn_sm80.qk_int8_sv_f16_accum_f16_attn(o, o, x, x, s, s, 1, 0, 2, 0.125, 0, m)
    with pytest.raises(NotImplementedError):
        ext._qattn_sm80.qk_int8_sv_int8_accum_f16_attn(o, o, x, x, s, s, 1, 0, 2, 0.125, 0, m)
    with pytest.raises(RuntimeError, match="Tensor Q must be on CUDA"):
        ext._rope.rope_permutation(x, x, torch.zeros(128), False)
    with pytest.raises(TypeError):
        ext._fused.quant_per_block_int8_cuda(x, o, s)       # neither overload
    import paroatten_amd
    import sys
    name = "paroattention_compiled_alias"
    try:
        paroatten_amd.install_alias(name, compiled=True)
        assert sys.modules[f"{name}._fused"] is ext._fused
        assert sys.modules[f"{name}.core"] is paroatten_amd.core
    finally:      # leave no alias behind for the rest of the session
        for mod in [m for m in sys.modules if m == name or m.startswith(name + ".")]:
            del sys.modules[mod]


@pytest.mark.gpu
def test_extension_matches_ctypes_mirrors_bit_for_bit(ext, dev):
    from paroatten_amd import _fused, _qattn_sm80, _rope
    B, H, N, D = 2, 3, 1000, 64
    nb = (N + 63) // 64
    q, k, v = (t.to(dev) for t in synth.make_qkv(B, H, N, D, torch.bfloat16, seed=3))
    km = k.mean(dim=2)

    def both(fn_name, make_outputs, args_of):
        outs = []
        for mod in (ext._fused, _fused):
            o = make_outputs()
            getattr(mod, fn_name)(*args_of(*o))
            outs.append(o)
        for a, b in zip(*outs):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), fn_name
        return outs[0]

    i8 = lambda: torch.empty(B, H, N, D, dtype=torch.int8, device=dev)
    f32 = lambda n: torch.empty(B, H, n, dtype=torch.float32, device=dev)
    q8, qs = both("quant_per_warp_int8_cuda", lambda: (i8(), f32(nb * 2)), lambda o, s: (q, o, s, 64, 32, 1))
    k8, ks = both("quant_per_block_int8_fuse_sub_mean_cuda", lambda: (i8(), f32(nb)), lambda o, s: (k, km, o, s, 64, 1))
    both("quant_per_block_int8_cuda", lambda: (i8(), f32(nb)), lambda o, s: (k, o, s, 64, 1))
    both("quant_per_block_int8_cuda", lambda: (i8(), f32((N + 127) // 128)), lambda o, s: (q, o, s, 0.18, 128, 1))
    both("sub_mean_cuda", lambda: (torch.empty(B, H, N, D, dtype=torch.float16, device=dev),), lambda o: (v, km, o, 1))
    padded = nb * 64
    (vt,) = both("transpose_pad_permute_cuda", lambda: (torch.empty(B, H, D, padded, dtype=v.dtype, device=dev),),
                 lambda o: (v, o, 1))
    f8 = lambda: torch.zeros(B, H, D, padded, dtype=torch.float8_e4m3fn, device=dev)
    hd = lambda: torch.empty(B, H, D, dtype=torch.float32, device=dev)
    both("mean_scale_fuse_quant_cuda", lambda: (f8(), hd(), hd()), lambda o, m, s: (vt, o, m, s, N, 448.0, 1))
    both("scale_fuse_quant_cuda", lambda: (f8(), hd()), lambda o, s: (vt, o, s, N, 448.0, 1))

    # the attention entry point: HND and NHD, with and without lse, [H,nb,nb] and [B,H,nb,nb] masks
    mask = synth.make_block_mask(H, nb, 0.5, seed=4).to(dev)
    for layout, lse_on, m in ((1, 1, mask), (1, 0, mask[None].expand(B, H, nb, nb).contiguous()), (0, 1, mask)):
        tr = (lambda t: t) if layout == 1 else (lambda t: t.transpose(1, 2).contiguous())
        res = []
        for mod in (ext._qattn_sm80, _qattn_sm80):
            out = torch.empty_like(tr(q))
            lse = mod.qk_int8_sv_f16_accum_f16_attn(tr(q8), tr(k8), tr(v), out, qs, ks, layout, 0, 2, D ** -0.5, lse_on, m)
            res.append((out, lse))
        assert torch.equal(res[0][0], res[1][0])
        assert res[0][1].shape == res[1][1].shape and torch.equal(res[0][1].cpu(), res[1][1].cpu())
        if not lse_on:
            assert res[0][1].numel() == 0 and not res[0][1].is_cuda     # the reference returns an empty CPU tensor
    # the flags the positional signature has no room for: a process-wide default of the compiled module
    from paroatten_amd import _lib
    assert ext._qattn_sm80.get_attention_flags() == 0
    for flags, kw in ((_lib.PARO_ATTN_PV_F16, dict(pv_f16=True)), (_lib.PARO_ATTN_EXACT_EXP, dict(exact_exp=True))):
        ext._qattn_sm80.set_attention_flags(flags)
        try:
            a, b = torch.empty_like(q), torch.empty_like(q)
            ext._qattn_sm80.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, a, qs, ks, 1, 0, 2, D ** -0.5, 0, mask)
        finally:
            ext._qattn_sm80.set_attention_flags(0)
        _qattn_sm80.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, b, qs, ks, 1, 0, 2, D ** -0.5, 0, mask, **kw)
        assert torch.equal(a, b), flags
    with pytest.raises(ValueError, match="tensor_layout must be 0 or 1"):
        ext._qattn_sm80.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, torch.empty_like(q), qs, ks, 7, 0, 2, 0.125, 0, mask)
    with pytest.raises(RuntimeError, match="Tensor sparse must have shape"):
        ext._qattn_sm80.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, torch.empty_like(q), qs, ks, 1, 0, 2, 0.125, 0, mask[:, :3].contiguous())
    # per-thread granularity: the reference's shape check (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:1034-1038), then the
    # same result as the ctypes mirror
    with pytest.raises(RuntimeError, match=r"Tensor query_scale must have shape .*\* 8"):
        ext._qattn_sm80.qk_int8_sv_f16_accum_f16_attn(q8, k8, v, torch.empty_like(q), qs, ks, 1, 0, 3, 0.125, 0, mask)
    from paroatten_amd import quant
    q8t, qst, k8t, kst = quant.per_thread_int8(q, k, km.unsqueeze(2))
    a, b = torch.empty_like(q), torch.empty_like(q)
    la = ext._qattn_sm80.qk_int8_sv_f16_accum_f16_attn(q8t, k8t, v, a, qst, kst, 1, 0, 3, D ** -0.5, 1, mask)
    lb = _qattn_sm80.qk_int8_sv_f16_accum_f16_attn(q8t, k8t, v, b, qst, kst, 1, 0, 3, D ** -0.5, 1, mask)
    assert torch.equal(a, b) and torch.equal(la, lb)

    # _rope.rope_permutation on the side stream torch is currently on
    g = torch.Generator(device=dev).manual_seed(5)
    Q = torch.randn(2, 6, 10, 256, generator=g, device=dev).half()
    K = torch.randn(2, 6, 10, 256, generator=g, device=dev).half()
    freq = torch.randn(128, generator=g, device=dev)
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        a = ext._rope.rope_permutation(Q, K, freq, True)
    side.synchronize()
    b = _rope.rope_permutation(Q, K, freq, True)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
