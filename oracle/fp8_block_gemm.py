"""TEST INFRASTRUCTURE ONLY - CPU oracle of the FP8 block-scaled GEMM path (torch on the host, fp32).

Each function restates one piece of the reference (paths relative to the DLBlas tree):

  e4m3fn_table / decode_e4m3fn   the OCP FP8 E4M3 ("fn": finite + NaN, no infinities) value table; what
                                 ``tensor.to(torch.float32)`` does in tests/kernels/test_fp8_gemm.py:59-60
  dequant_ref                    the closed form of the test's ``gt`` fixture, tests/kernels/test_fp8_gemm.py:33-68
                                 = the arithmetic of fp8_gemm_kernel, dlblas/kernels/fp8_gemm.py:49-60
  dequant_ref_blocked            the same fixture in its original block-looped shape (:57-65)
  quant_act_group / _1x128       per_token_group_quant_fp8 (any group size / 128), dlblas/kernels/fp8.py:44-51,108-182
  quant_weight_128x128           128 x 128 block quantiser; the reference has none in the package, the scheme
                                 (block amax / 448) is that of its test data builder,
                                 tests/kernels/test_fused_moe_v2.py:35-60
  grouped_contiguous_ref         deep_gemm.m_grouped_fp8_gemm_nt_contiguous as used at
                                 dlblas/kernels/fused_moe_v3.py:235-245,307-308 (deep_gemm v2.1.1.post3 is pinned
                                 in prose only, dlblas/layers/README.md:2, and is not vendored)
  grouped_masked_ref             deep_gemm.m_grouped_fp8_gemm_nt_masked as used at
                                 dlblas/layers/moe/ep_moe.py:180-197,218-224

How each one is pinned (tests/test_oracle.py):
  decode        exhaustively, all 256 codes, against torch's own float8_e4m3fn -> float32 cast and against the
                format definition evaluated with exact rationals
  dequant_ref   against dequant_ref_blocked (independent loop structure), against the C restatement in
                fp8_gemm_oracle.c (independent decode + accumulation), against exact integer arithmetic on
                small-integer inputs, against one-hot inputs (output = one dequantised weight column), with
                negative scales, ragged N and K, M = 1
  quantisers    invariants that fix the formula: |q| <= 448, a group's amax maps to +-448, reconstruction error
                bounded by half an e4m3 ulp of the scaled value, all-zero group -> eps scale; RTNE ties checked
                against a brute-force nearest-value search
  grouped       PARITY UNPINNED against deep_gemm itself (absent from the reference tree and this image; the
                reference has no test at that boundary).  Pinned to the dense oracle by brute force per expert,
                which is what the call sites' shapes and the public deep_gemm contract state.
"""
from fractions import Fraction

import numpy as np
import torch

BLOCK = 128
E4M3_MAX = 448.0


# ---------------------------------------------------------------------------------------------------------------
# e4m3fn decode
# ---------------------------------------------------------------------------------------------------------------
def e4m3fn_value(code: int) -> Fraction:
    """Exact value of one e4m3fn code as a rational (NaN codes 0x7f / 0xff raise ValueError)."""
    sign = -1 if code & 0x80 else 1
    exp = (code >> 3) & 0xF
    man = code & 0x7
    if exp == 0xF and man == 0x7:
        raise ValueError('NaN')
    if exp == 0:
        return sign * Fraction(man, 8) * Fraction(1, 2**6)
    mag = (1 + Fraction(man, 8)) * (Fraction(2)**(exp - 7))
    return sign * mag


def e4m3fn_table() -> np.ndarray:
    """float32[256]: value of every e4m3fn code (NaN for 0x7f and 0xff)."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        try:
            value = float(e4m3fn_value(code))
            out[code] = np.float32(-0.0 if (code == 0x80) else value)  # a Fraction cannot carry the sign of zero
        except ValueError:
            out[code] = np.float32('nan')
    return out


_TABLE = None


def decode_e4m3fn(t: torch.Tensor) -> torch.Tensor:
    """float8_e4m3fn (or its uint8 bit pattern) -> float32 through the value table."""
    global _TABLE
    if _TABLE is None:
        _TABLE = torch.from_numpy(e4m3fn_table())
    bits = t.view(torch.uint8) if t.dtype != torch.uint8 else t
    return _TABLE[bits.long()]


# ---------------------------------------------------------------------------------------------------------------
# dense GEMM
# ---------------------------------------------------------------------------------------------------------------
def _expand_a_scale(a_s: torch.Tensor, K: int) -> torch.Tensor:
    return a_s.repeat_interleave(BLOCK, dim=-1)[..., :K]


def _expand_b_scale(b_s: torch.Tensor, N: int, K: int) -> torch.Tensor:
    return b_s.repeat_interleave(BLOCK, dim=0).repeat_interleave(BLOCK, dim=1)[:N, :K]


def dequant_ref(a_q, a_s, b_q, b_s, out_dtype=torch.float32) -> torch.Tensor:
    """Dequantise both operands to fp32, multiply, cast once: ``(a_q * a_s) @ (b_q * b_s).T``.

    a_q [..., K] e4m3fn, a_s [..., ceil(K/128)] f32, b_q [N, K] e4m3fn, b_s [ceil(N/128), ceil(K/128)] f32.
    """
    K = a_q.shape[-1]
    N = b_q.shape[0]
    a = decode_e4m3fn(a_q).reshape(-1, K) * _expand_a_scale(a_s.float().reshape(-1, a_s.shape[-1]), K)
    b = decode_e4m3fn(b_q) * _expand_b_scale(b_s.float(), N, K)
    c = a @ b.t()
    return c.reshape(*a_q.shape[:-1], N).to(out_dtype)


def dequant_ref_blocked(a_q, a_s, b_q, b_s, out_dtype=torch.float32) -> torch.Tensor:
    """Block-looped form: for every (K block i, N block j) add ``(A_i @ B_ji.T) * (a_s[:, i] * b_s[j, i])``."""
    M, K = a_q.shape
    N = b_q.shape[0]
    a = decode_e4m3fn(a_q)
    b = decode_e4m3fn(b_q)
    c = torch.zeros(M, N, dtype=torch.float32)
    for i in range(-(-K // BLOCK)):
        ks = slice(i * BLOCK, min((i + 1) * BLOCK, K))
        for j in range(-(-N // BLOCK)):
            ns = slice(j * BLOCK, min((j + 1) * BLOCK, N))
            scale = a_s[:, i:i + 1].float() * b_s[j, i].float()
            c[:, ns] += (a[:, ks] @ b[ns, ks].t()) * scale
    return c.to(out_dtype)


# ---------------------------------------------------------------------------------------------------------------
# quantisers
# ---------------------------------------------------------------------------------------------------------------
def quant_act_group(x: torch.Tensor, group_size: int, eps: float = 1e-10):
    """Per row and group of ``group_size`` consecutive elements (any divisor of K, dlblas/kernels/fp8.py:35-51):
    ``s = max(amax, eps) / 448``, ``q = clamp(x / s, -448, 448)`` cast RTNE to e4m3fn.

    x [..., K] with K % group_size == 0.  Returns (q e4m3fn [..., K], s f32 [..., K / group_size]).
    """
    assert x.shape[-1] % group_size == 0
    xf = x.float().reshape(*x.shape[:-1], x.shape[-1] // group_size, group_size)
    amax = xf.abs().amax(dim=-1, keepdim=True).clamp_min(eps)
    s = amax / E4M3_MAX
    q = (xf / s).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return q.reshape(x.shape), s.squeeze(-1).contiguous()


def quant_act_1x128(x: torch.Tensor, eps: float = 1e-10):
    """quant_act_group at the group size of the block-scaled GEMM: (q e4m3fn [..., K], s f32 [..., K/128])."""
    return quant_act_group(x, BLOCK, eps)


def quant_weight_128x128(w: torch.Tensor, eps: float = 1e-10):
    """Per 128 x 128 block (ragged at the N and K edges): ``s = max(amax, eps) / 448``, same cast as above.

    w [N, K].  Returns (q e4m3fn [N, K], s f32 [ceil(N/128), ceil(K/128)]).
    """
    N, K = w.shape
    nb, kb = -(-N // BLOCK), -(-K // BLOCK)
    wf = torch.zeros(nb * BLOCK, kb * BLOCK, dtype=torch.float32)
    wf[:N, :K] = w.float()
    blocks = wf.reshape(nb, BLOCK, kb, BLOCK)
    amax = blocks.abs().amax(dim=(1, 3), keepdim=True).clamp_min(eps)
    s = amax / E4M3_MAX
    q = (blocks / s).clamp(-E4M3_MAX, E4M3_MAX).reshape(nb * BLOCK, kb * BLOCK)[:N, :K]
    return q.to(torch.float8_e4m3fn).contiguous(), s.reshape(nb, kb).contiguous()


# ---------------------------------------------------------------------------------------------------------------
# grouped GEMMs (brute force over experts on top of dequant_ref)
# ---------------------------------------------------------------------------------------------------------------
def grouped_contiguous_ref(a_q, a_s, w_q, w_s, out: torch.Tensor, m_indices: torch.Tensor) -> torch.Tensor:
    """Rows whose 128-row block starts with expert g >= 0 get the dense product with expert g's weights; blocks
    starting with a negative index keep the previous content of ``out``.  Returns ``out`` (modified in place)."""
    M = a_q.shape[0]
    for r0 in range(0, M, BLOCK):
        g = int(m_indices[r0])
        if g < 0:
            continue
        rows = slice(r0, min(r0 + BLOCK, M))
        out[rows] = dequant_ref(a_q[rows], a_s[rows], w_q[g], w_s[g], out.dtype)
    return out


def grouped_masked_ref(a_q, a_s, w_q, w_s, out: torch.Tensor, masked_m: torch.Tensor) -> torch.Tensor:
    """For every expert g only rows [0, masked_m[g]) are computed and written.  Returns ``out``."""
    G, M_max = a_q.shape[0], a_q.shape[1]
    for g in range(G):
        m = max(0, min(int(masked_m[g]), M_max))
        if m:
            out[g, :m] = dequant_ref(a_q[g, :m], a_s[g, :m], w_q[g], w_s[g], out.dtype)
    return out


# ---------------------------------------------------------------------------------------------------------------
# error metrics
# ---------------------------------------------------------------------------------------------------------------
def max_rel_err(out: torch.Tensor, ref: torch.Tensor, floor_frac: float = 1e-3) -> float:
    """max |out - ref| / max(|ref|, floor_frac * rms(ref)): relative error with a floor so that outputs that
    cancel to ~0 are judged against the typical magnitude of the result instead of against zero."""
    o, r = out.double().flatten(), ref.double().flatten()
    if r.numel() == 0:
        return 0.0
    rms = float(torch.sqrt(torch.mean(r * r)))
    denom = torch.clamp(r.abs(), min=max(floor_frac * rms, 1e-30))
    return float(((o - r).abs() / denom).max())


def similarity_gap(x: torch.Tensor, y: torch.Tensor) -> float:
    """1 - 2<x, y> / (|x|^2 + |y|^2): the global similarity metric of dlblas/utils/utils.py:113-140."""
    x, y = x.double(), y.double()
    denom = float((x * x + y * y).sum())
    if denom == 0:
        return 0.0
    return 1.0 - 2.0 * float((x * y).sum()) / denom
