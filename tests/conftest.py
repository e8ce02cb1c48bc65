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
