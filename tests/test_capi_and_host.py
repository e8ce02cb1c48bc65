"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header
declares, reports its architecture, and the Python mirrors reject bad arguments with the
reference's exception types before anything touches a GPU."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols(header="paroatten.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(paro_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import paroatten_amd._lib as L
    lib = L.load()
    names = _declared_symbols()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/paroatten.h but not exported"
        assert n in L.SIGNATURES, f"{n} has no ctypes signature"
    assert set(L.SIGNATURES) == set(names)
    assert lib.paro_abi_version() == 2
    assert lib.paro_build_arch() == b"gfx950"
    raw = ctypes.CDLL(str(L.LIB_PATH))
    assert raw.paro_abi_version() == 2


def test_measurement_aids_live_outside_the_product_library():
    """include/paroatten_diag.h (bench.py --mfma-ceiling / --proxy-ceiling) is a library of its own: every symbol
    it declares is exported there, none of them by libparoatten_hip.so, and its argument checks answer on the CPU."""
    import paroatten_amd._lib as L
    names = _declared_symbols("paroatten_diag.h")
    assert len(names) >= 7 and all(n.startswith("paro_diag_") for n in names)
    diag = ctypes.CDLL(str(L.LIB_PATH.parent / "libparoatten_diag.so"))
    product = ctypes.CDLL(str(L.LIB_PATH))
    for n in names:
        assert hasattr(diag, n), f"{n} declared in include/paroatten_diag.h but not exported"
        assert not hasattr(product, n), f"{n} leaked into the product library"
        assert n not in L.SIGNATURES
    assert not any(n.startswith("paro_diag_") for n in _declared_symbols())
    diag.paro_diag_last_error.restype = ctypes.c_char_p
    assert diag.paro_diag_attn_proxy(7, None, None, None, 1, 1, 4, None) == -1
    assert b"level" in diag.paro_diag_last_error()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.c_void_p(ctypes.addressof(buf))
    assert diag.paro_diag_attn_proxy(0, p, p, p, 1, 1, 70000, None) == -1      # block list entries are 16 bits
    assert diag.paro_diag_attn_proxy_w64(0, p, p, p, p, 1, 3, 8, None) == -2     # odd iteration count


def test_size_queries_need_no_gpu():
    import paroatten_amd._lib as L
    lib = L.load()
    assert lib.paro_v_fp8_bytes(2, 48, 17776, 64) == 2 * 48 * 278 * 64 * 64
    # statistics: 3 values per chunk of 1024 tokens and channel; residual sums: 2 per 64-token tile
    assert lib.paro_v_fp8_partial_floats(1, 1, 1024, 64) == (3 + 16 * 2) * 64
    assert lib.paro_v_fp8_partial_floats(1, 1, 1025, 128) == (2 * 3 + 17 * 2) * 128
    ws = lib.paro_attn_workspace_bytes(2, 48, 17776, 64)
    assert ws >= lib.paro_v_fp8_bytes(2, 48, 17776, 64) and ws % 256 == 0


def test_c_abi_argument_errors_without_gpu():
    """argument validation happens before any launch: codes and messages come back on CPU"""
    import paroatten_amd._lib as L
    lib = L.load()
    rc = lib.paro_quant_int8(None, 0, None, None, None, 1, 1, 64, 64, 0, 0, 64, 0, 0, 0, 0, 64, 0, 0, 32, 2, 0, 0.0, None)
    assert rc == L.PARO_ERR_RUNTIME and b"null" in lib.paro_last_error()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 255) & ~255)
    rc = lib.paro_quant_int8(p, 0, None, p, p, 1, 1, 64, 96, 0, 0, 96, 0, 0, 0, 0, 96, 0, 0, 32, 2, 0, 0.0, None)
    assert rc == L.PARO_ERR_INVALID_VALUE and lib.paro_last_error() == b"Unsupported head dim: 96"
    with pytest.raises(ValueError, match="Unsupported head dim: 96"):
        L.check(rc)
    rc = lib.paro_quant_int8(p, 0, None, p, p, 1, 1, 64, 64, 0, 0, 64, 0, 0, 0, 0, 64, 0, 0, 48, 2, 0, 0.0, None)
    assert rc == L.PARO_ERR_INVALID_VALUE
    rc = lib.paro_quant_int8(p, 0, None, p, p, 1, 1, 64, 64, 0, 0, 64, 0, 0, 0, 0, 64, 0, 0, 32, 1, 0, 0.0, None)
    assert rc == L.PARO_ERR_RUNTIME and b"do not cover" in lib.paro_last_error()
    rc = lib.paro_transpose_pad_permute(p, p, 0, 1, 1, 100, 64, 0, 0, 64, 0, 0, 64, None)
    assert rc == L.PARO_ERR_RUNTIME and b"ceil64(num_tokens) = 128" in lib.paro_last_error()
    assert lib.paro_transpose_pad_permute(p, p, 0, 1, 1, 100, 80, 0, 0, 80, 0, 0, 128, None) == L.PARO_ERR_INVALID_VALUE
    rc = lib.paro_channel_quant_fp8(p, 0, p, None, p, 1, 1, 64, 100, 64, 448.0, 0, 0, 64, 0, 0, 64, 0, 0, 0, 0, None)
    assert rc == L.PARO_ERR_RUNTIME and b"shorter than ceil64" in lib.paro_last_error()
    rc = lib.paro_channel_quant_fp8(p, 0, p, None, p, 1, 1, 64, 100, 128, 0.0, 0, 0, 128, 0, 0, 128, 0, 0, 0, 0, None)
    assert rc == L.PARO_ERR_INVALID_VALUE and b"scale_max" in lib.paro_last_error()
    rc = lib.paro_permute_inv(p, p, 0, p, 1, 1, 100, 64, 10, 3, 5, 7, 0, 0, 64, 0, 0, 64, None)
    assert rc == L.PARO_ERR_RUNTIME and b"does not equal the token count" in lib.paro_last_error()
    # per-thread scales go with neither the float16 P.V product nor the score dump
    rc = lib.paro_attn_sparse_fwd(p, p, p, p, p, p, p, p, 0, p, 0, None, None, 1, 1, 1, 64, 64, 64,
                                  0, 0, 64, 0, 0, 64, 0, 0, 64, 0.125, 0,
                                  L.PARO_ATTN_PV_F16 | L.PARO_ATTN_QK_PER_THREAD, None)
    assert rc == L.PARO_ERR_UNSUPPORTED and b"per-thread" in lib.paro_last_error()
    with pytest.raises(NotImplementedError):
        L.check(rc)
    rc = lib.paro_qk_int8_sv_f16_attn(p, p, p, 0, p, 0, p, p, p, 0, None, p, 1 << 30, 1, 1, 1, 64, 64, 64,
                                      0, 0, 64, 0, 0, 64, 0, 0, 64, 0, 0, 64, 1, 0, 4, 0.125, 1, 0, None)
    assert rc == L.PARO_ERR_INVALID_VALUE and b"granularity" in lib.paro_last_error()
    rc = lib.paro_qk_int8_sv_f16_attn(p, p, p, 0, p, 0, p, p, p, 0, None, p, 16, 1, 1, 1, 64, 64, 64,
                                      0, 0, 64, 0, 0, 64, 0, 0, 64, 0, 0, 64, 1, 0, 2, 0.125, 1, 0, None)
    assert rc == L.PARO_ERR_RUNTIME and b"workspace" in lib.paro_last_error()
    rc = lib.paro_qk_int8_sv_f16_attn(p, p, p, 0, p, 0, p, p, p, 0, None, p, 1 << 30, 1, 1, 1, 64, 64, 64,
                                      0, 0, 64, 0, 0, 64, 0, 0, 64, 0, 0, 64, 7, 0, 2, 0.125, 1, 0, None)
    assert rc == L.PARO_ERR_INVALID_VALUE and lib.paro_last_error() == b"tensor_layout must be 0 or 1"


def test_python_mirrors_reject_cpu_tensors_and_bad_flags():
    from paroatten_amd import _fused, _qattn_sm80, _rope, core, quant
    x = torch.zeros(1, 1, 64, 64, dtype=torch.float16)
    o = torch.zeros(1, 1, 64, 64, dtype=torch.int8)
    s = torch.zeros(1, 1, 2)
    with pytest.raises(RuntimeError, match="Tensor input must be on CUDA"):
        _fused.quant_per_warp_int8_cuda(x, o, s, 64, 32, 1)
    with pytest.raises(ValueError, match="Unsupported block_size 48"):
        _fused.quant_per_block_int8_cuda(x, o, s, 48, 1)
    with pytest.raises(ValueError, match="Unsupported warp_block_size 8"):
        _fused.quant_per_warp_int8_cuda(x, o, s, 64, 8, 1)
    with pytest.raises(ValueError, match="Unknown tensor layout"):
        quant.per_warp_int8(x, x, tensor_layout="DNH")
    with pytest.raises(RuntimeError, match="Tensor query must be on CUDA"):
        _qattn_sm80.qk_int8_sv_f16_accum_f16_attn(o, o, x, x, s, s, 1, 0, 2, 0.125, 0, torch.ones(1, 1, 1, 1, dtype=torch.bool))
    with pytest.raises(NotImplementedError):
        _qattn_sm80.qk_int4_sv_f16_accum_f16_attn()
    with pytest.raises(RuntimeError, match="Tensor input must be on CUDA"):
        _fused.transpose_pad_permute_cuda(x, x, 1)
    with pytest.raises(RuntimeError, match="Tensor input must be on CUDA"):
        _fused.mean_scale_fuse_quant_cuda(x, x, s, s, 64, 448.0, 1)
    with pytest.raises(RuntimeError, match="Tensor input must be on CUDA"):
        _fused.scale_fuse_quant_cuda(x, x, s, 64, 448.0, 1)
    with pytest.raises(AssertionError, match="must be on cuda"):
        core.paroattn_qk_int8_pv_fp16_cuda(x, x, x, torch.ones(1, 1, 1, dtype=torch.bool))
    with pytest.raises(RuntimeError):
        _rope.rope_permutation(x, x, torch.zeros(128), False)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    import paroatten_amd._lib as L
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setenv("PAROATTEN_LIB", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError, match="no fallback"):
        L.load()
    monkeypatch.delenv("PAROATTEN_LIB")
    L.load()


def test_mask_generator_contract():
    from paroatten_amd import synth
    for nb, dens in ((64, 0.5), (278, 0.3), (40, 0.2)):
        m = synth.make_block_mask(3, nb, dens, seed=1)
        assert m.shape == (3, nb, nb) and m.dtype == torch.bool
        target = max(int(round(dens * nb * nb)), int(((torch.arange(nb)[:, None] - torch.arange(nb)[None]).abs() <= 2).sum()))
        assert (m.sum(dim=(1, 2)) == target).all()
        i = torch.arange(nb)
        assert m[:, i, i].all() and m[:, i[:-2], i[:-2] + 2].all() and m[:, i[2:], i[2:] - 2].all()
    assert torch.equal(synth.make_block_mask(2, 16, 0.4, seed=5), synth.make_block_mask(2, 16, 0.4, seed=5))
    w = synth.make_window_mask(2, 40, 0.2)
    assert w.shape == (2, 40, 40) and (w.sum(dim=2) == 8).all() and w[:, torch.arange(40), torch.arange(40)].all()
    assert ((w[0].int().diff(dim=1) != 0).sum(dim=1) <= 2).all()      # one contiguous run per row
    plan = synth.make_permute_plan(4, 48, seed=0)
    assert plan["permute"].shape == (4, 48) and int(plan["permute"].min()) >= 0 and int(plan["permute"].max()) <= 5


def test_new_entry_points_validate_without_gpu():
    """the one-pass preparation, the folded inverse permutation and the mask bit kernels reject bad
    arguments before any launch"""
    import paroatten_amd._lib as L
    lib = L.load()
    assert lib.paro_mask_bits_bytes(0) == 0 and lib.paro_mask_bits_bytes(9) == 2 and lib.paro_mask_bits_bytes(-3) == 0
    assert lib.paro_mask_pack(None, None, 0, None) == L.PARO_OK            # nothing to do
    assert lib.paro_mask_pack(None, None, 16, None) == L.PARO_ERR_RUNTIME and b"null" in lib.paro_last_error()
    assert lib.paro_mask_unpack(None, None, -1, None) == L.PARO_ERR_INVALID_VALUE
    buf = ctypes.create_string_buffer(8192)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 255) & ~255)
    odd = ctypes.c_void_p(p.value + 4)
    assert lib.paro_mask_unpack(odd, p, 64, None) == L.PARO_ERR_RUNTIME and b"aligned" in lib.paro_last_error()
    # the larger of the K-mean partials (70 chunks of 256) and the V statistics + residual sums (18 chunks of 1024, 278 tiles)
    assert lib.paro_prep_workspace_bytes(2, 48, 17776, 64) == 2 * 48 * (18 * 3 + 278 * 2) * 64 * 4

    def prep(D=64, N=128, grid=(2, 8, 8), n_text=0, q=p, ws=p, ws_bytes=1 << 20):
        return lib.paro_rope_permute_quant_fwd(q, p, p, 0, None, None, p, None, p, p, p, p, p, p, p, ws, ws_bytes,
                                               1, 1, N, D, n_text, grid[0], grid[1], grid[2],
                                               N * D, N * D, D, N * D, N * D, D, N * D, N * D, D, 0, 0, 1, None)
    assert prep(D=96) == L.PARO_ERR_INVALID_VALUE and lib.paro_last_error() == b"Unsupported head dim: 96"
    assert prep(grid=(2, 8, 9)) == L.PARO_ERR_RUNTIME and b"does not equal the token count" in lib.paro_last_error()
    assert prep(q=None) == L.PARO_ERR_RUNTIME and b"null" in lib.paro_last_error()
    assert prep(ws_bytes=16) == L.PARO_ERR_RUNTIME and b"workspace" in lib.paro_last_error()

    rc = lib.paro_attn_sparse_unpermute_fwd(p, p, p, p, p, p, p, p, 0, p, 0, None, 1, 1, 1, 128, 128, 64,
                                            8192, 8192, 64, 8192, 8192, 64, 8192, 8192, 64, 0.125, 0, 0,
                                            None, 0, 2, 8, 8, None)
    assert rc == L.PARO_ERR_RUNTIME and b"null orders" in lib.paro_last_error()
    rc = lib.paro_attn_sparse_unpermute_fwd(p, p, p, p, p, p, p, p, 0, p, 0, None, 1, 1, 1, 128, 128, 64,
                                            8192, 8192, 64, 8192, 8192, 64, 8192, 8192, 64, 0.125, 0, 0,
                                            p, 1, 2, 8, 8, None)
    assert rc == L.PARO_ERR_RUNTIME and b"does not equal the token count" in lib.paro_last_error()
    rc = lib.paro_rope_k_mean(p, 0, p, None, p, p, 1 << 20, 1, 1, 128, 64, 0, 2, 8, 8, 8192, 8192, 64, 64, 64, None)
    assert rc == L.PARO_ERR_RUNTIME and b"cos and sin" in lib.paro_last_error()


def test_size_limits_are_rejected_without_gpu():
    """batch * heads beyond the launch-grid range, slices beyond the 32-bit buffer offsets and key
    lists beyond the local data share come back as errors, not launches"""
    import paroatten_amd._lib as L
    lib = L.load()
    buf = ctypes.create_string_buffer(8192)
    p = ctypes.c_void_p((ctypes.addressof(buf) + 255) & ~255)
    N, D = 128, 64
    rc = lib.paro_rope_permute_fwd(p, None, None, p, None, None, 0, None, None, p, 1024, 64, N, D, 0, 2, 8, 8,
                                   64 * N * D, N * D, D, 64 * N * D, N * D, D, None)
    assert rc == L.PARO_ERR_RUNTIME and b"exceeds 65535" in lib.paro_last_error()
    rc = lib.paro_quant_int8(p, 0, None, p, p, 1, 70000, N, D, 0, N * D, D, 0, 0, 0, N * D, D, 0, 2, 64, 2, 0, 0.0, None)
    assert rc == L.PARO_ERR_RUNTIME and b"exceeds 65535" in lib.paro_last_error()
    # one-pass preparation: a token stride that puts the last row of a head 2 GiB away
    big = 1 << 24
    rc = lib.paro_rope_permute_quant_fwd(p, p, p, 0, None, None, p, None, p, p, p, p, p, p, p, p, 1 << 20,
                                         1, 1, N, D, 0, 2, 8, 8, 0, 0, big, N * D, N * D, D, N * D, N * D, D,
                                         0, 0, 1, None)
    assert rc == L.PARO_ERR_RUNTIME and b"2 GiB" in lib.paro_last_error()
    # attention: 30 million keys = 468 750 blocks, far more than the 65 535 a block index can hold
    Nk = 30_000_000
    rc = lib.paro_attn_sparse_fwd(p, p, p, p, p, p, p, p, 0, p, 0, None, None, 1, 1, 1, 64, Nk, D,
                                  64 * D, 64 * D, D, Nk * D, Nk * D, D, 64 * D, 64 * D, D, 0.125, 0, 0, None)
    assert rc == L.PARO_ERR_RUNTIME and b"exceeds 65535 blocks" in lib.paro_last_error()
    # 2 million keys fit the block index but not the list in the local data share
    Nk = 2_000_000
    rc = lib.paro_attn_sparse_fwd(p, p, p, p, p, p, p, p, 0, p, 0, None, None, 1, 1, 1, 64, Nk, D,
                                  64 * D, 64 * D, D, Nk * D, Nk * D, D, 64 * D, 64 * D, D, 0.125, 0, 0, None)
    assert rc == L.PARO_ERR_RUNTIME and b"local data share" in lib.paro_last_error()


def test_import_paroattention_resolves_by_itself():
    """Callers of the reference do `import paroattention` / `from paroattention.cogvideox import ...`
    (example/pipeline_cogvideox.py:15-16, paroattention/__init__.py:1-5 of the reference): a fresh interpreter
    finds the same names here without any set-up call."""
    import subprocess
    import sys
    code = (
        "import paroattention, paroatten_amd\n"
        "assert paroattention is paroatten_amd\n"
        "import paroattention.core, paroattention.quant, paroattention.cogvideox, paroattention.wan\n"
        "import paroattention.prefetch_utils, paroattention.prefetch_wan, paroattention.utils\n"
        "import paroattention._qattn_sm80, paroattention._fused, paroattention._rope\n"
        "from paroattention import paroattn, paroattn_qk_int8_pv_fp16_cuda, PARO_CogVideoXAttnProcessor2_0, "
        "PARO_WanAttnProcessor2_0\n"
        "from paroattention.cogvideox import PARO_CogVideoXAttnProcessor2_0 as C\n"
        "from paroattention.prefetch_utils import TimestepCallback, SparseMaskPrefetchStream\n"
        "from paroattention.prefetch_wan import TimestepCallback as TW\n"
        "from paroattention.quant import per_block_int8, per_warp_int8, sub_mean, per_channel_fp8\n"
        "assert C is PARO_CogVideoXAttnProcessor2_0 and paroattention.core is paroatten_amd.core\n"
        "print('ok')\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip() == "ok", r.stderr[-2000:]


def test_wan_model_names_subclass_diffusers_when_it_is_there():
    """paroattention/__init__.py:4-5 exports PARO_WanTransformerBlock and PARO_WanTransformer3DModel; here they are
    subclasses of diffusers' classes built on first use.  With a stand-in `diffusers` (two classes of the same
    names and shape: a block with `attn1.set_processor`, a model with `.blocks`) every attn1 ends up with a
    PARO_WanAttnProcessor2_0; without diffusers the names raise ImportError that names the alternative."""
    import subprocess
    import sys
    code = (
        "import sys, types\n"
        "import paroattention\n"
        "try:\n"
        "    paroattention.PARO_WanTransformer3DModel\n"
        "    raise SystemExit('expected ImportError')\n"
        "except ImportError as e:\n"
        "    assert 'set_paro_processors' in str(e)\n"
        "class Attn:\n"
        "    def __init__(self): self.processor = 'stock'\n"
        "    def set_processor(self, p): self.processor = p\n"
        "class WanTransformerBlock:\n"
        "    def __init__(self, dim=8): self.dim = dim; self.attn1 = Attn(); self.attn2 = Attn()\n"
        "class WanTransformer3DModel:\n"
        "    def __init__(self, num_layers=3): self.blocks = [WanTransformerBlock() for _ in range(num_layers)]\n"
        "tw = types.ModuleType('diffusers.models.transformers.transformer_wan')\n"
        "tw.WanTransformerBlock, tw.WanTransformer3DModel = WanTransformerBlock, WanTransformer3DModel\n"
        "for name in ('diffusers', 'diffusers.models', 'diffusers.models.transformers'):\n"
        "    m = types.ModuleType(name); m.__path__ = []; sys.modules[name] = m\n"
        "sys.modules['diffusers.models.transformers.transformer_wan'] = tw\n"
        "sys.modules['diffusers.models.transformers'].transformer_wan = tw\n"
        "from paroattention import PARO_WanTransformer3DModel, PARO_WanTransformerBlock, PARO_WanAttnProcessor2_0\n"
        "from paroattention.wan import PARO_WanTransformer3DModel as M2\n"
        "assert M2 is PARO_WanTransformer3DModel and issubclass(PARO_WanTransformer3DModel, WanTransformer3DModel)\n"
        "model = PARO_WanTransformer3DModel(num_layers=4)\n"
        "assert len(model.blocks) == 4\n"
        "assert all(isinstance(b.attn1.processor, PARO_WanAttnProcessor2_0) for b in model.blocks)\n"
        "assert all(b.attn2.processor == 'stock' for b in model.blocks)\n"
        "assert len({id(b.attn1.processor) for b in model.blocks}) == 4\n"
        "blk = PARO_WanTransformerBlock(dim=16)\n"
        "assert blk.dim == 16 and isinstance(blk.attn1.processor, PARO_WanAttnProcessor2_0)\n"
        "print('ok')\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip() == "ok", r.stderr[-2000:]
