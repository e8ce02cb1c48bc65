import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda:0")


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.double().flatten()
    b = b.double().flatten()
    return float((a @ b) / (a.norm() * b.norm()).clamp_min(1e-300))


ATOL = 2e-2          # the benchmark's tolerance on attention outputs (fp16)
FP8_STEP = 2.0 ** -4   # one e4m3 rounding (3 mantissa bits) at its worst, relative


def assert_attention_close(o: torch.Tensor, o_ref: torch.Tensor, a_ref: torch.Tensor, cos: float = 0.999, what: str = "",
                           frac_one_step: float = 1e-3):
    """The one tolerance rule for attention outputs at any shape.  `a_ref` is the oracle's attention with |V| in
    place of V (same weights p): A_ij = sum_j p_ij |v_j|, the scale an output element is built on.  P and V enter
    the product as e4m3 codes, each up to 2^-4 off in relative terms, so the error of an element is relative to
    A, not to the element itself (which cancellation can make arbitrarily small):
        every element:              |o - o_ref| <= ATOL + 2 * 2^-4 * A   (both roundings at their worst: two
                                                                          comparable keys of opposite sign)
        all but 1e-3 of them:       |o - o_ref| <= ATOL + 2^-4 * A       (one rounding at its worst; tests whose
                                    data is built so that a few keys dominate most rows state a larger fraction)
        cosine(o, o_ref) >= 0.999.
    At the benchmark shapes, where long rows average V down to |o| ~ 0.05 (A ~ 0.8 / sqrt(n) scale), the A terms
    are below a few 1e-3 and the rule is the flat atol 2e-2; on short rows and on rows that a few keys dominate
    (outputs of order 1) it is what FP8 operands can promise."""
    e = (o.float() - o_ref.float()).abs()
    a = a_ref.float()
    worst = float((e - (ATOL + 2 * FP8_STEP * a)).max())
    assert worst <= 0.0, f"{what}: |o - o_ref| exceeds {ATOL} + 2^-3 * sum p|v| by {worst:.4g} (max abs err {float(e.max()):.4g})"
    frac = float((e > ATOL + FP8_STEP * a).float().mean())
    assert frac <= frac_one_step, f"{what}: {frac:.3g} of the elements exceed {ATOL} + 2^-4 * sum p|v|"
    c = cosine(o, o_ref)
    assert c >= cos, f"{what}: cosine {c}"


def untile_v8(v8: torch.Tensor, B: int, H: int, N: int, D: int) -> torch.Tensor:
    """FP8 V tiles as paro_v_fp8_pack writes them ([B,H,nb][D/32][2][64 lanes][16 bytes]: byte r of
    lane l of piece (dt, mt) = token 64*kb + 32*mt + 8*(r//4) + 4*(l//32) + r%4, channel 32*dt + l%32)
    -> uint8 [B, H, nb*64, D] in token order (CPU)."""
    nb = (N + 63) // 64
    t = v8.view(torch.uint8).flatten().cpu().reshape(B, H, nb, D // 32, 2, 2, 32, 4, 4)
    #                                            dims: b  h  kb   dt   mt lh  l32 g  q
    # token inside the tile = 32*mt + 8*g + 4*lh + q ; channel = 32*dt + l32
    return t.permute(0, 1, 2, 4, 7, 5, 8, 3, 6).reshape(B, H, nb * 64, D).contiguous()


def v8_offset_expected(v: torch.Tensor, tok_bytes: torch.Tensor, v_scale: torch.Tensor) -> torch.Tensor:
    """What the attention epilogue has to add back per channel for the codes `tok_bytes` (uint8
    [B,H,>=N,D] in token order) of v [B,H,N,D] under scales v_scale [B,H,D]:
    mean_n(v - v_scale * e4m3(code)), in float64."""
    N = v.shape[2]
    deq = tok_bytes[:, :, :N].view(torch.float8_e4m3fn).double() * v_scale.double().cpu()[:, :, None, :]
    return (v.double().cpu() - deq).mean(dim=2)
