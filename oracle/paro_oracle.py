"""CPU restatement of the PAROAttention hot path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module; the product package must never route through it.

Every function restates, in plain torch on the CPU, what one piece of the reference
computes (file:line of /root/reference cited per function).  The CUDA extensions of the
reference cannot be built without nvcc and an NVIDIA GPU, and the reference holds no golden
vectors for this path, so each function is pinned by what the mathematics fixes (closed
forms, brute force on tiny inputs, reduction to a library routine) in tests/test_oracle_*.py.

Pinning status
  quant_int8 / per_warp_int8 / per_block_int8 : pinned (closed-form KAT of bench/test.py,
        invariants, brute force)
  per_thread_scale_index / per_thread_int8    : pinned (the index law against an enumeration of the
        reference kernel's accumulator lanes, :112-116 and :129-133 of its .cu; the quantiser reduces to
        quant_int8 on tokens regrouped so that every group is contiguous)
  qk_int32                                    : pinned (int64 einsum brute force)
  sparse_attention                            : pinned (reduces to softmax(mask)@V library
        routine, dense SDPA special case, empty-row and K-smoothing invariants, lse closed form; with
        per-thread scales: reduces to the per-warp result for scales that are constant per group, and to
        fp64 softmax attention on tensors dequantised row by row)
  permute maps / permute_qk / permute_attn_out: pinned (torch.permute library routine, the
        reference's literal tables, inverse∘forward = id)
  rope_wan                                    : pinned (complex rotation, norm, composition)
  rope_cog (cos/sin table convention of diffusers' get_3d_rotary_pos_embed) : pinned (the
        rotation by complex multiplication and norm preservation; the table by closed forms
        evaluated in Python floats: 16/24/24 channel groups that each depend on one grid axis,
        angle = pos * theta^(-2i/dim_group) on both channels of pair i, and an independent
        second construction in paroatten_amd/rope.py compared bit for bit)
  per_channel_fp8                             : pinned against torch.float8_e4m3fn casting
  transpose_pad_permute                       : pinned (torch.transpose + pad library routines; the
        within-16 order is stated twice by the reference, as a formula in the kernel and as a
        literal list in a docstring, and the two are checked against each other)
  channel_quant_fp8                           : pinned (float64 statistics, torch.float8_e4m3fn
        casting; reduces to per_channel_fp8 when the token count is a multiple of 16)
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch

LOG2E = 1.44269504  # the literal the reference uses (paroattention/quant.py:94, core.py:214)

# paroattention/cogvideox.py:38-45  (index -> order of the (F,H,W) axes)
PERMUTATIONS = (
    (0, 1, 2),  # 0: FHW
    (0, 2, 1),  # 1: FWH
    (1, 2, 0),  # 2: HWF
    (1, 0, 2),  # 3: HFW
    (2, 1, 0),  # 4: WHF
    (2, 0, 1),  # 5: WFH
)
# paroattention/cogvideox.py:85-92
PERMUTATIONS_INV = (
    (0, 1, 2),
    (0, 2, 1),
    (2, 0, 1),
    (1, 0, 2),
    (2, 1, 0),
    (1, 2, 0),
)


# ----------------------------------------------------------------------------------------
# INT8 quantisation  (csrc/fused/fused.cu:64-198, hosts :512-592, :594-682, :685-768)
# ----------------------------------------------------------------------------------------
def quant_int8(
    x: torch.Tensor,
    group: int,
    n_groups: Optional[int] = None,
    mean: Optional[torch.Tensor] = None,
    sm_scale: Optional[float] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Symmetric INT8 quantisation of x [B,H,N,D] (HND) in groups of `group` tokens.

    Follows QuantInt8Kernel (fused.cu:64-198): x = float(in); x -= float(mean[b,h,:]) if a
    mean is given (:119-126); x *= sm_scale if given (:128-135); tokens >= N read as 0
    (:137-144); amax = max(1e-7, max|x|) (:147-156); scale = amax / 127 (:163);
    q = rint_ties_even(x * (127 / amax)) saturated to int8 (:168-186,
    numeric_conversion.cuh:137-142).  IEEE fp32 arithmetic (the CUDA build's fast-math
    rounding is not part of the specification).
    """
    B, H, N, D = x.shape
    if n_groups is None:
        n_groups = (N + group - 1) // group
    xf = x.to(torch.float32)
    if mean is not None:
        xf = xf - mean.to(torch.float32).reshape(B, H, 1, D)
    if sm_scale is not None:
        xf = xf * torch.tensor(sm_scale, dtype=torch.float32)
    npad = n_groups * group
    if npad > N:
        xf = torch.nn.functional.pad(xf, (0, 0, 0, npad - N))
    g = xf.reshape(B, H, n_groups, group * D)
    amax = g.abs().amax(dim=-1).clamp_min(torch.tensor(1e-7, dtype=torch.float32))
    scale = amax / torch.tensor(127.0, dtype=torch.float32)
    inv = torch.tensor(127.0, dtype=torch.float32) / amax
    q = torch.round(g * inv.unsqueeze(-1)).clamp_(-128, 127).to(torch.int8)
    q = q.reshape(B, H, npad, D)[:, :, :N].contiguous()
    return q, scale


def per_warp_int8(q, k, km=None, BLKQ=128, WARPQ=32, BLKK=64):
    """paroattention/quant.py:105-180 (HND): Q per WARPQ tokens, K per BLKK tokens.
    q_scale has ceil(N/BLKQ)*(BLKQ/WARPQ) entries (:170)."""
    nq = q.shape[2]
    n_groups_q = ((nq + BLKQ - 1) // BLKQ) * (BLKQ // WARPQ)
    q8, qs = quant_int8(q, WARPQ, n_groups=n_groups_q)
    if km is not None:
        km = km.reshape(k.shape[0], k.shape[1], k.shape[3])  # quant.py:174-176 squeeze
    k8, ks = quant_int8(k, BLKK, mean=km)
    return q8, qs, k8, ks


def per_thread_scale_index(n: int, is_key: bool) -> torch.Tensor:
    """Scale index of each of n tokens at the per-thread granularity (qk_quant_gran 3) of
    qk_int_sv_f16_attn_kernel with CTA_Q = CTA_K = WARP_K = 64, WARP_Q = 32.  A thread of the m16n8
    accumulator tiles holds rows lane/4 and lane/4 + 8 of every 16-row tile and columns 2*(lane%4),
    2*(lane%4)+1 of every 8-column tile, and reads q scale `warp*8 + lane/4` and k scale
    `block*4 + lane%4` (csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:112-116, 129-133).  So query token r uses
    scale (r//32)*8 + r%8 and key token c uses scale (c//64)*4 + (c%8)//2."""
    t = torch.arange(n)
    if is_key:
        return (t // 64) * 4 + (t % 8) // 2
    return (t // 32) * 8 + t % 8


def quant_int8_per_thread(x: torch.Tensor, is_key: bool, mean: Optional[torch.Tensor] = None):
    """The arithmetic of quant_int8 on the token groups of per_thread_scale_index.  The reference has no
    quantiser of this granularity (paroattention/core.py:204-205 calls the per-block one, whose scales the
    kernel's shape check :1034-1038 rejects): this is the quantiser its kernel's indexing implies.
    Returns (int8 [B,H,N,D], scale [B,H,ceil(N/64)*(4 if is_key else 16)])."""
    B, H, N, D = x.shape
    xf = x.to(torch.float32)
    if mean is not None:
        xf = xf - mean.to(torch.float32).reshape(B, H, 1, D)
    npad = (N + 63) // 64 * 64
    if npad > N:
        xf = torch.nn.functional.pad(xf, (0, 0, 0, npad - N))   # tokens >= N read as 0, whatever the mean
    idx = per_thread_scale_index(npad, is_key)
    n_scales = npad // 64 * (4 if is_key else 16)
    tok_amax = xf.abs().amax(dim=-1)
    amax = torch.zeros(B, H, n_scales, dtype=torch.float32)
    amax = amax.scatter_reduce(2, idx.expand(B, H, npad), tok_amax, reduce="amax", include_self=True)
    amax = amax.clamp_min(torch.tensor(1e-7, dtype=torch.float32))
    scale = amax / torch.tensor(127.0, dtype=torch.float32)
    inv = torch.tensor(127.0, dtype=torch.float32) / amax
    q = torch.round(xf * inv[:, :, idx].unsqueeze(-1)).clamp_(-128, 127).to(torch.int8)
    return q[:, :, :N].contiguous(), scale


def per_thread_int8(q, k, km=None):
    """Q and K at the per-thread granularity (HND); km as in per_warp_int8."""
    if km is not None:
        km = km.reshape(k.shape[0], k.shape[1], k.shape[3])
    q8, qs = quant_int8_per_thread(q, False)
    k8, ks = quant_int8_per_thread(k, True, mean=km)
    return q8, qs, k8, ks


def per_block_int8(q, k, km=None, BLKQ=128, BLKK=64, sm_scale=None):
    """paroattention/quant.py:22-103 (HND): folds sm_scale*1.44269504 into Q (:91-96)."""
    D = q.shape[-1]
    if sm_scale is None:
        sm_scale = D ** -0.5
    sm_scale = sm_scale * LOG2E
    q8, qs = quant_int8(q, BLKQ, sm_scale=sm_scale)
    if km is not None:
        km = km.reshape(k.shape[0], k.shape[1], k.shape[3])
    k8, ks = quant_int8(k, BLKK, mean=km)
    return q8, qs, k8, ks


# ----------------------------------------------------------------------------------------
# Integer QK^T   (csrc/qattn/attn_utils.cuh:202-324: int8 x int8 -> int32, exact)
# ----------------------------------------------------------------------------------------
def qk_int32(q8: torch.Tensor, k8: torch.Tensor) -> torch.Tensor:
    """S[b,h,i,j] = sum_d q8[b,h,i,d]*k8[b,h,j,d] as int32.  Computed by an fp64 GEMM,
    exact because |S| <= 127*127*128 < 2^24 (tests pin it against an int64 einsum)."""
    s = torch.matmul(q8.to(torch.float64), k8.to(torch.float64).transpose(-1, -2))
    return s.to(torch.int32)


# ----------------------------------------------------------------------------------------
# Block-sparse quantised attention
#   csrc/qattn/qk_int_sv_f16_cuda_sm80.cu:100-133 (scale indexing), :222,:268 (mask indexing),
#   :136-169 (m=-5e6, d=1, O=0 => a row with no kept block outputs 0),
#   csrc/qattn/attn_utils.cuh:355-381 (columns >= kv_len excluded), :383-488 (online softmax),
#   :786-840 (normalisation), :711-723 of the .cu (lse = log2(d) + m, base 2)
# ----------------------------------------------------------------------------------------
def expand_block_mask(mask: torch.Tensor, nq: int, nk: int, block: int = 64) -> torch.Tensor:
    """bool [.., nbq, nbk] -> bool [.., nq, nk] (kron with ones(block,block), cropped)."""
    m = mask.repeat_interleave(block, dim=-2).repeat_interleave(block, dim=-1)
    return m[..., :nq, :nk]


def sparse_attention(
    q8: torch.Tensor,
    k8: torch.Tensor,
    v: torch.Tensor,
    q_scale: torch.Tensor,
    k_scale: torch.Tensor,
    mask: torch.Tensor,
    sm_scale: float,
    warp_q: int = 32,
    blk_k: int = 64,
    is_causal: bool = False,
    out_dtype: torch.dtype = torch.float16,
    compute_dtype: torch.dtype = torch.float32,
    q_chunk: int = 2048,
    per_thread: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Intended semantics of qk_int8_sv_f16_accum_f16_attn (HND, gran = per_warp; with per_thread=True
    gran = per_thread: the scales of row i and column j are those of per_thread_scale_index):

      s_ij = (sum_d q8_id k8_jd) * q_scale[b,h,i//warp_q] * k_scale[b,hk,j//blk_k] * sm_scale
      J(i) = { j < N : mask[b,h,i//64,j//64] }  (and j <= i if causal)
      o_i  = sum_{j in J(i)} softmax_j(s_ij) v_j ;  J(i) empty => o_i = 0
      lse_i (base 2, as the kernel returns it) = log2 sum_{j in J(i)} exp(s_ij)

    V is rounded to fp16 first (paroattention/core.py:208 `v.to(torch.float16)`).  The
    reference's internal rounding points (fp16 P, fp16 accumulators, approx exp2/rcp) are
    not reproduced: they are implementation detail, the tolerance of the parity tests
    (atol 2e-2, cosine >= 0.999) covers them.  An all-masked row gives 0 and lse = -inf
    (the reference's finite stand-in for it is m0 = -5e6).
    Returns (o [B,H,N,D] out_dtype, lse_base2 [B,H,N] fp32).
    """
    B, H, N, D = q8.shape
    Hk, Nk = k8.shape[1], k8.shape[2]
    groups = H // Hk
    vf = v.to(torch.float16).to(compute_dtype)
    o = torch.zeros(B, H, N, D, dtype=compute_dtype)
    lse = torch.full((B, H, N), float("-inf"), dtype=torch.float32)
    col = torch.arange(Nk)
    for b in range(B):
        for h in range(H):
            hk = h // groups
            kf = k8[b, hk].to(compute_dtype)
            if per_thread:
                ksc = k_scale[b, hk].to(compute_dtype)[per_thread_scale_index(Nk, True)]
            else:
                ksc = k_scale[b, hk].to(compute_dtype).repeat_interleave(blk_k)[:Nk]
            for i0 in range(0, N, q_chunk):
                i1 = min(N, i0 + q_chunk)
                qf = q8[b, h, i0:i1].to(compute_dtype)
                s = qf @ kf.T  # exact integers (< 2^24) in fp32/fp64
                row = torch.arange(i0, i1)
                qsc = q_scale[b, h].to(compute_dtype)[per_thread_scale_index(N, False)[row] if per_thread else row // warp_q]
                s = s * (qsc[:, None] * ksc[None, :]) * sm_scale
                keep = mask[b, h][row // 64][:, col // 64]
                if is_causal:
                    keep = keep & (col[None, :] <= row[:, None])
                s = s.masked_fill(~keep, float("-inf"))
                mx = s.amax(dim=-1, keepdim=True)
                mx = torch.where(torch.isinf(mx), torch.zeros_like(mx), mx)
                p = torch.exp(s - mx)
                d = p.sum(dim=-1, keepdim=True)
                empty = d == 0
                o[b, h, i0:i1] = torch.where(empty, torch.zeros_like(d), 1.0 / d) * (p @ vf[b, hk])
                l = (torch.log(d) + mx).squeeze(-1) * LOG2E
                lse[b, h, i0:i1] = torch.where(empty.squeeze(-1), torch.full_like(l, float("-inf")), l).float()
    return o.to(out_dtype), lse


# ----------------------------------------------------------------------------------------
# Token permutation   (paroattention/cogvideox.py:22-62, :64-110; wan.py:25-111)
# ----------------------------------------------------------------------------------------
def permute_index_map(grid: Sequence[int], order_id: int) -> torch.Tensor:
    """new_of_old[old] for one head: the index law of permute_qk.  With sizes S=(F,H,W),
    coordinates c=(f,h,w) of `old = (f*H + h)*W + w` and order p = PERMUTATIONS[order_id]:
    new = (c[p0]*S[p1] + c[p1])*S[p2] + c[p2], and out[new] = in[old]."""
    F, Hh, W = grid
    p = PERMUTATIONS[order_id]
    S = (F, Hh, W)
    old = torch.arange(F * Hh * W)
    c = (old // (Hh * W), (old // W) % Hh, old % W)
    return (c[p[0]] * S[p[1]] + c[p[1]]) * S[p[2]] + c[p[2]]


def permute_qk(query, key, value, permute_plan, i_block, grid, n_text):
    """Restates permute_qk (cogvideox.py:22-62) in its own reshape/permute form, out of
    place, with (F,H,W) and the text length as arguments instead of literals."""
    F, Hh, W = grid
    outs = []
    order_idx = permute_plan["permute"][i_block]
    for t in (query, key, value):
        BS, NH, NT, ND = t.shape
        n_img = NT - n_text
        assert n_img == F * Hh * W
        o = t.clone()
        for ih in range(NH):
            p = PERMUTATIONS[int(order_idx[ih])]
            ext = (0, p[0] + 1, p[1] + 1, p[2] + 1, 4)
            o[:, ih, n_text:, :] = (
                t[:, ih, n_text:, :].reshape(BS, F, Hh, W, ND).permute(*ext).reshape(BS, n_img, ND)
            )
        outs.append(o)
    return tuple(outs)


def permute_attn_out(attn_out, permute_plan, i_block, grid, n_text):
    """Restates permute_attn_out (cogvideox.py:64-110): view the image part in the
    permuted shape, permute back with PERMUTATIONS_INV."""
    F, Hh, W = grid
    BS, NH, NT, ND = attn_out.shape
    n_img = NT - n_text
    order_idx = permute_plan["permute"][i_block]
    o = attn_out.clone()
    full = (BS, F, Hh, W, ND)
    for ih in range(NH):
        p = PERMUTATIONS[int(order_idx[ih])]
        pinv = PERMUTATIONS_INV[int(order_idx[ih])]
        ext = (0, p[0] + 1, p[1] + 1, p[2] + 1, 4)
        ext_inv = (0, pinv[0] + 1, pinv[1] + 1, pinv[2] + 1, 4)
        shape = tuple(full[e] for e in ext)
        o[:, ih, n_text:, :] = (
            attn_out[:, ih, n_text:, :].reshape(*shape).permute(*ext_inv).reshape(BS, n_img, ND)
        )
    return o


# ----------------------------------------------------------------------------------------
# RoPE
# ----------------------------------------------------------------------------------------
def rope_apply_cog(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """diffusers apply_rotary_emb(x, (cos, sin)) with use_real=True, unbind_dim=-1, as the
    reference calls it on the image tokens (paroattention/cogvideox.py:167-172):
    x_rot = stack([-x_imag, x_real]) interleaved; out = (x.float()*cos + x_rot.float()*sin)
    cast to x.dtype.  cos/sin are [N, D] fp32."""
    xr, xi = x.reshape(*x.shape[:-1], -1, 2).unbind(-1)
    x_rot = torch.stack([-xi, xr], dim=-1).flatten(-2)
    return (x.float() * cos + x_rot.float() * sin).to(x.dtype)


def rope_apply_wan(x: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """paroattention/wan.py:161-167: complex multiply in float64, cast back.
    freqs complex128 [1,1,N,D/2]."""
    xc = torch.view_as_complex(x.to(torch.float64).unflatten(3, (-1, 2)))
    return torch.view_as_real(xc * freqs).flatten(3, 4).type_as(x)


def rope_1d_freqs(dim: int, length: int, theta: float = 10000.0) -> torch.Tensor:
    """angles[pos, i] = pos * theta^(-2i/dim), float64, [length, dim/2]
    (get_1d_rotary_pos_embed as called at wan.py:497-499)."""
    inv = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64)[: dim // 2] / dim))
    return torch.outer(torch.arange(length, dtype=torch.float64), inv)


def rope_table_wan(head_dim: int, grid: Sequence[int], theta: float = 10000.0) -> torch.Tensor:
    """WanRotaryPosEmbed (wan.py:482-522): t/h/w split = D-4*(D//6), 2*(D//6), 2*(D//6)
    channels; complex128 [1,1,F*H*W,D/2] gathered per (f,h,w)."""
    F, Hh, W = grid
    h_dim = w_dim = 2 * (head_dim // 6)
    t_dim = head_dim - h_dim - w_dim
    af = rope_1d_freqs(t_dim, F, theta).view(F, 1, 1, -1).expand(F, Hh, W, -1)
    ah = rope_1d_freqs(h_dim, Hh, theta).view(1, Hh, 1, -1).expand(F, Hh, W, -1)
    aw = rope_1d_freqs(w_dim, W, theta).view(1, 1, W, -1).expand(F, Hh, W, -1)
    ang = torch.cat([af, ah, aw], dim=-1).reshape(1, 1, F * Hh * W, -1)
    return torch.polar(torch.ones_like(ang), ang)


def rope_table_cog(head_dim: int, grid: Sequence[int], theta: float = 10000.0):
    """CogVideoX 3-D table in the documented diffusers convention: channels split
    t/h/w = D/4, 3D/8, 3D/8, every frequency repeated twice (repeat_interleave 2), cos/sin
    fp32 [F*H*W, D].  The reference only consumes the finished (cos, sin) pair
    (cogvideox.py:167-172); the convention (third-party diffusers get_3d_rotary_pos_embed, no
    version pinned by the reference, not importable here) is pinned by closed forms in
    tests/test_oracle_permute_rope.py (test_rope_cog_table_closed_form)."""
    F, Hh, W = grid
    dt, dh, dw = head_dim // 4, head_dim // 8 * 3, head_dim // 8 * 3
    af = rope_1d_freqs(dt, F, theta).repeat_interleave(2, dim=1)
    ah = rope_1d_freqs(dh, Hh, theta).repeat_interleave(2, dim=1)
    aw = rope_1d_freqs(dw, W, theta).repeat_interleave(2, dim=1)
    ang = torch.cat(
        [
            af.view(F, 1, 1, -1).expand(F, Hh, W, -1),
            ah.view(1, Hh, 1, -1).expand(F, Hh, W, -1),
            aw.view(1, 1, W, -1).expand(F, Hh, W, -1),
        ],
        dim=-1,
    ).reshape(F * Hh * W, head_dim)
    return ang.cos().float(), ang.sin().float()


# ----------------------------------------------------------------------------------------
# V -> FP8   (paroattention/quant.py:224-293, csrc/fused/fused.cu:316-427)
# ----------------------------------------------------------------------------------------
def per_channel_fp8(v: torch.Tensor, scale_max: float = 448.0, smooth_v: bool = True):
    """Per-(b,h,channel) e4m3 quantisation of V [B,H,N,D]: vm = mean over the N tokens,
    scale = max|v - vm| / scale_max, v8 = e4m3_rne_satfinite((v - vm) * (scale_max / max|v - vm|)).  Returned in
    token-major form [B,H,N,D] (the reference's transposed+shuffled storage,
    fused.cu:262-313, is an NVIDIA fragment layout and not part of the arithmetic).
    Deviation kept on purpose: the mean divides by N, not by ceil16(N) (fused.cu:335,381)."""
    vf = v.to(torch.float32)
    if smooth_v:
        vm = vf.mean(dim=2)
        vf = vf - vm.unsqueeze(2)
    else:
        vm = None
    amax = vf.abs().amax(dim=2)
    scale = amax / scale_max
    # fused.cu:399,414: multiply by recp_scale = scale_max / amax (a constant channel gives 0, not NaN)
    # a tensor / tensor quotient: a Python scalar divided by a tensor is evaluated as reciprocal-times-
    # scalar, which rounds twice
    recp = torch.where(amax > 0, torch.full_like(amax, scale_max) / amax, torch.zeros_like(amax))
    v8 = (vf * recp.unsqueeze(2)).clamp(-scale_max, scale_max).to(torch.float8_e4m3fn)
    return v8, scale, vm


# paroattention/quant.py:231-234 (docstring of per_channel_fp8): position i of every group of 16
# tokens holds token V_SHUFFLE16[i]
V_SHUFFLE16 = (0, 1, 8, 9, 2, 3, 10, 11, 4, 5, 12, 13, 6, 7, 14, 15)


def shuffle16_position_of(r: int) -> int:
    """where TransposePadPermuteKernel puts token r of a group of 16 (csrc/fused/fused.cu:287-291:
    smem_load_row = (r / 8) * 2 + ((r / 2) % 4) * 4 + r % 2)."""
    return (r // 8) * 2 + ((r // 2) % 4) * 4 + r % 2


def transpose_pad_permute(v: torch.Tensor) -> torch.Tensor:
    """transpose_pad_permute_cuda for the HND layout (csrc/fused/fused.cu:262-313, 850-923):
    [B,H,N,D] -> [B,H,D,ceil64(N)], zero padding, tokens inside every group of 16 reordered."""
    B, H, N, D = v.shape
    padded = (N + 63) // 64 * 64
    x = torch.nn.functional.pad(v.transpose(2, 3), (0, padded - N))          # [B,H,D,padded]
    src = torch.arange(padded).view(-1, 16)[:, list(V_SHUFFLE16)].reshape(-1)   # out[i] = in[src[i]]
    return x[..., src].contiguous()


def channel_quant_fp8(x: torch.Tensor, num_tokens: int, scale_max: float = 448.0, sub_mean: bool = True):
    """MeanScaleKernel behind mean_scale_fuse_quant_cuda / scale_fuse_quant_cuda
    (csrc/fused/fused.cu:316-427): x [B,H,D,L] 16-bit rows.  Statistics over the first
    n16 = ceil16(num_tokens) entries (:335-336: the zero padding takes part, and the mean divides by
    n16, :381); amax = max(|max - mean|, |min - mean|) (:385); scale = amax / scale_max (:393);
    codes for the first ceil64(num_tokens) entries: e4m3((x - mean) * (scale_max / amax)) (:399-421).
    Returns (codes float8 [B,H,D,ceil64], scale f32 [B,H,D], mean f32 [B,H,D] or None).  A constant row
    gives zero codes (the reference divides by zero there)."""
    n16 = (num_tokens + 15) // 16 * 16
    n64 = (num_tokens + 63) // 64 * 64
    xf = x.to(torch.float32)
    head = xf[..., :n16]
    mean = (head.double().sum(dim=-1) / n16).float() if sub_mean else torch.zeros(x.shape[:-1])
    amax = torch.maximum((head.amax(dim=-1) - mean).abs(), (head.amin(dim=-1) - mean).abs())
    scale = amax / scale_max
    recp = torch.where(amax > 0, torch.full_like(amax, scale_max) / amax, torch.zeros_like(amax))   # one rounding
    codes = ((xf[..., :n64] - mean.unsqueeze(-1)) * recp.unsqueeze(-1)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return codes, scale, (mean if sub_mean else None)


# ----------------------------------------------------------------------------------------
# The whole path, as the processors chain it (cogvideox.py:167-227)
# ----------------------------------------------------------------------------------------
def paro_path(q, k, v, mask, permute_plan, i_block, grid, n_text, cos=None, sin=None,
              smooth_k=True, sm_scale=None):
    """RoPE (image tokens) -> per-head permutation -> per-warp INT8 quant (K optionally
    mean-smoothed, core-API style km = mean over tokens) -> block-sparse attention ->
    inverse permutation.  Returns the output in the original token order."""
    D = q.shape[-1]
    if sm_scale is None:
        sm_scale = D ** -0.5
    if cos is not None:
        q = q.clone()
        k = k.clone()
        q[:, :, n_text:] = rope_apply_cog(q[:, :, n_text:], cos, sin)
        k[:, :, n_text:] = rope_apply_cog(k[:, :, n_text:], cos, sin)
    qp, kp, vp = permute_qk(q, k, v, permute_plan, i_block, grid, n_text)
    km = kp.float().mean(dim=2, keepdim=True).to(kp.dtype) if smooth_k else None
    q8, qs, k8, ks = per_warp_int8(qp, kp, km=km, BLKQ=64, WARPQ=32, BLKK=64)
    o, _ = sparse_attention(q8, k8, vp, qs, ks, mask, sm_scale, out_dtype=q.dtype)
    return permute_attn_out(o, permute_plan, i_block, grid, n_text)
