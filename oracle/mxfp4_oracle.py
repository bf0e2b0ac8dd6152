"""CPU restatement (torch, CPU tensors only) of ALTO's MXFP4 arithmetic.

THIS IS TEST INFRASTRUCTURE.  It is the checker for the HIP kernels, never a
code path of the product: only ``tests/``, ``__graft_entry__.smoke`` and the
``cpu_baseline`` leg of ``bench.py`` import it.

Each function cites the reference lines it follows (paths relative to the
reference checkout):

* scale rule        alto/kernels/fp4/mxfp4/mxfp_quantization.py:28-95
                    tests/unittest/mxfp4/utils.py:320-348
* E2M1 encode RNE   alto/kernels/fp4/fp4_common/triton_fp4_ops.py:24-47,62-95
                    tests/unittest/mxfp4/utils.py:34-146
* E2M1 encode SR    alto/kernels/fp4/fp4_common/triton_fp4_ops.py:49-61,79-80
* E2M1 decode       alto/kernels/fp4/fp4_common/triton_fp4_ops.py:98-134
                    tests/unittest/mxfp4/utils.py:151-235
* pack / unpack     alto/kernels/fp4/mxfp4/mxfp_quantization.py:115,186
                    tests/unittest/mxfp4/utils.py:265-282
* host layouts      alto/kernels/fp4/mxfp4/mxfp_quantization.py:410-484,487-545
* Hadamard          alto/kernels/hadamard_transform/transform.py:98-142
                    alto/kernels/hadamard_transform/hadamard.py:63-87,130-161
                    alto/kernels/hadamard_transform/matrix.py:129-163
* GEMM              alto/kernels/fp4/mxfp4/mxfp_linear.py:142-255
* linear fwd/bwd    alto/kernels/fp4/mxfp4/mxfp_linear.py:265-570
* grouped GEMM      alto/kernels/fp4/mxfp4/mxfp_grouped_gemm/cg_forward.py:200-303
                    alto/kernels/fp4/mxfp4/mxfp_grouped_gemm/cg_backward.py:398-930
* offs -> indices   alto/kernels/dsgemm_utils.py:96-112

Parity status of each function (what pins it, since the reference holds no
golden files for this path) is recorded in ``tests/test_oracle_*.py``:
closed forms, exhaustive enumeration against brute force, counting identities
for stochastic rounding and a second, scalar pure-Python-int model in
``oracle/scalar_model.py``.

Parity unpinned (no check available without running the reference's Triton kernels on gfx950):
* ``clip_mode="dynamic"`` (``block_scales``) on bf16 tensors: the ORDER of the fp32 sums of the block statistics and
  whether the final multiply-add is contracted are Triton's choice in the reference, and its own test does not hold the
  bf16 case bit-equal to anything (tests/unittest/mxfp4/test_mxfp_quantization.py:69-70).  On fp32 tensors the branch IS
  pinned: tests/golden/reference_vectors.npz holds the outputs of the reference's PyTorch twin, which that test asserts
  bit-equal to the Triton kernel, and closed-form scale bytes are checked in tests/test_oracle_pins.py.
* the accumulation order inside ``tl.dot_scaled`` / ``v_mfma_scale`` (GEMMs are compared with a tolerance).

Two deliberate departures from the reference (both are inputs the reference
draws from hidden state and this build takes explicitly):

* stochastic rounding consumes a caller-supplied tensor of 32 random bits per
  element (``rand_bits``, same shape as the input; element ``x[i, j]`` uses
  ``rand_bits[i, j]`` whatever the quantisation axis) instead of an in-kernel
  Philox stream with tile-local offsets;
* the randomized Hadamard transform consumes explicit ``signs`` (32 values of
  +-1) and ``perm`` (a permutation of 0..31) instead of a class-level
  ``torch.Generator``; its fp32 summation order is FIXED (see ``rht_left``),
  where the reference leaves it to the BLAS backend.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

BLOCK = 32
SQRT32_F32 = 5.656854152679443  # float32(sqrt(32)); transform.py:113 keeps a float64 0-dim tensor, the divide runs in fp32

__all__ = [
    "BLOCK", "SQRT32_F32", "E2M1_GRID",
    "e8m0_from_absmax", "block_scales", "encode_e2m1_rne", "encode_e2m1_sr", "decode_e2m1",
    "pack_nibbles", "unpack_nibbles", "quantize", "dequantize",
    "hadamard_matrix", "rht_left", "rht_left_dense", "rht", "rht_dense",
    "gemm_ref", "linear_forward_ref", "linear_backward_ref",
    "indices_from_offsets", "grouped_gemm_ref", "grouped_gemm_dx_ref", "grouped_gemm_dw_ref",
    "rel_frobenius", "dge_bwd_ref", "weight_grid_values", "E2M1_BREAK_POINTS",
]

E2M1_GRID = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


# --------------------------------------------------------------------------- scale (Q1)
def e8m0_from_absmax(absmax: torch.Tensor, use_uos: bool = False, target_max_pow2: int = 2) -> torch.Tensor:
    """E8M0 byte from a block absmax held in the INPUT dtype (bf16 or fp32).

    mxfp_quantization.py:73-94: the absmax is bit-cast to int16 (bf16, 7
    mantissa bits) or int32 (fp32, 23 bits); a quarter of the mantissa range is
    added so that mantissas >= 1.75 carry into the exponent, the 9 bits above
    the mantissa are taken, 2 is subtracted, and the result is clamped below
    at 1 (never above).
    """
    assert absmax.dtype in (torch.bfloat16, torch.float32)
    if use_uos:
        # mxfp_quantization.py:75-78
        a = absmax.float()
        s = torch.ceil(torch.log2(a / 7.25))
        s = torch.where(a == 0, torch.ones_like(s), s) + 127
        s = torch.where(s < 1, torch.ones_like(s), s)
        return s.to(torch.uint8)
    if absmax.dtype == torch.float32:
        bits = absmax.contiguous().view(torch.int32).to(torch.int64)
        mbits = 23
    else:
        bits = absmax.contiguous().view(torch.int16).to(torch.int64)
        mbits = 7
    e = ((bits + (1 << (mbits - 2))) & (0x1FF << mbits)) >> mbits
    s = e - target_max_pow2
    s = torch.clamp(s, min=1)
    return s.to(torch.uint8)


def _block_view(x2d: torch.Tensor, is_2d_block: bool) -> torch.Tensor:
    """[R, C] -> [..., 32] (1D) or [R/32, C/32, 1024] (2D) view used for the block reduction."""
    R, C = x2d.shape
    if is_2d_block:
        return x2d.reshape(R // BLOCK, BLOCK, C // BLOCK, BLOCK).transpose(1, 2).reshape(R // BLOCK, C // BLOCK, BLOCK * BLOCK)
    return x2d.reshape(R, C // BLOCK, BLOCK)


def block_scales(x2d: torch.Tensor, is_2d_block: bool = False, clip_mode: str = "none", use_uos: bool = False) -> torch.Tensor:
    """Scales of a quant-axis-last 2D tensor: [R, C/32] (1D) or [R/32, C/32] (2D). mxfp_quantization.py:28-95."""
    blk = _block_view(x2d, is_2d_block)
    if clip_mode == "dynamic":
        # mxfp_quantization.py:54-59,65-70.  The squares are rounded to the input dtype (an elementwise product of bf16
        # tensors is bf16), the sums run in fp32 (Triton promotes bf16 reductions).  The ORDER of the fp32 sums is left
        # to Triton's reduction in the reference; it is fixed here: the 32 elements of a block row in index order, then
        # (2D) the 32 row sums in row order.  Multiply and add of the max_abs formula round separately, as in the
        # reference's PyTorch twin (tests/unittest/mxfp4/utils.py:320-325).  Parity with the Triton kernel's own order of
        # additions is unpinned (it could not be run); the HIP kernel follows THIS order bit for bit.
        R, C = x2d.shape
        xr = x2d.reshape(R, C // BLOCK, BLOCK)
        xf = xr.float()
        sq = (xr * xr).float()
        s1 = torch.zeros(R, C // BLOCK, dtype=torch.float32)
        s2 = torch.zeros(R, C // BLOCK, dtype=torch.float32)
        for i in range(BLOCK):
            s1 = s1 + xf[..., i]
            s2 = s2 + sq[..., i]
        n = float(BLOCK)
        if is_2d_block:
            s1 = s1.reshape(R // BLOCK, BLOCK, C // BLOCK)
            s2 = s2.reshape(R // BLOCK, BLOCK, C // BLOCK)
            t1 = torch.zeros(R // BLOCK, C // BLOCK, dtype=torch.float32)
            t2 = torch.zeros(R // BLOCK, C // BLOCK, dtype=torch.float32)
            for j in range(BLOCK):
                t1 = t1 + s1[:, j]
                t2 = t2 + s2[:, j]
            s1, s2, n = t1, t2, float(BLOCK * BLOCK)
        mean_sq = s2 / n
        mean = s1 / n
        std = torch.sqrt(mean_sq - mean * mean)
        absmax = (torch.tensor(2.92247856 / 6.0, dtype=torch.float32) * std + torch.tensor(1e-8, dtype=torch.float32)).to(x2d.dtype)
        return e8m0_from_absmax(absmax, use_uos=use_uos, target_max_pow2=0)
    absmax = blk.abs().amax(dim=-1)  # exact in any dtype
    return e8m0_from_absmax(absmax, use_uos=use_uos)


# --------------------------------------------------------------------------- encode (Q2, Q4)
def _split_sign(q: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    assert q.dtype == torch.float32
    bits = q.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    sign = bits & 0x80000000
    mag_bits = bits ^ sign
    mag = mag_bits.to(torch.int32).view(torch.float32)  # < 2^31 so the int32 cast keeps the pattern
    return sign, mag_bits, mag


def encode_e2m1_rne(q: torch.Tensor) -> torch.Tensor:
    """fp32 (already divided by the scale) -> 4-bit E2M1 code, round-to-nearest-even. triton_fp4_ops.py:38-47,62-93."""
    sign, mag_bits, mag = _split_sign(q)
    saturate = mag >= 6.0
    denormal = (~saturate) & (mag < 1.0)
    # subnormal lane: the fp32 add of 2^22 performs the RNE to multiples of 0.5
    magic = torch.tensor(0x4A800000, dtype=torch.int32).view(torch.float32)
    den = (mag + magic).view(torch.int32).to(torch.int64) - 0x4A800000
    den = den & 0xFF
    # normal lane
    mant_odd = (mag_bits >> 22) & 1
    nor = (mag_bits + ((1 - 127) << 23) + 0x1FFFFF + mant_odd) & 0xFFFFFFFF
    nor = (nor >> 22) & 0xFF
    code = torch.full_like(mag_bits, 7)
    code = torch.where(saturate, code, torch.where(denormal, den, nor))
    code = code | (sign >> 28)
    return code.to(torch.uint8)


def _as_u32(rand_bits: torch.Tensor) -> torch.Tensor:
    """Random bits as int64 values in [0, 2^32); accepts uint32 / int32 / int64 storage."""
    if rand_bits.dtype == torch.uint32:
        return rand_bits.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    if rand_bits.dtype == torch.int32:
        return rand_bits.to(torch.int64) & 0xFFFFFFFF
    assert rand_bits.dtype == torch.int64
    return rand_bits & 0xFFFFFFFF


def encode_e2m1_sr(q: torch.Tensor, rand_bits: torch.Tensor) -> torch.Tensor:
    """fp32 -> E2M1 code with stochastic rounding from 32 explicit random bits per element.

    triton_fp4_ops.py:49-61,79-80.  Subnormal lane (|q| < 1): the compare is
    ``rand <= threshold`` (unsigned), thresholds ``trunc(|q| * 2^33)`` below
    0.5 and ``trunc((2|q| - 1) * 2^32)`` from 0.5 (the Python constants
    2**33-2 and 2**32-1 round to 2^33 and 2^32 in fp32).  Normal lane: the low
    22 random bits are added under the kept mantissa bit and the sum is
    truncated.
    """
    sign, mag_bits, mag = _split_sign(q)
    r = _as_u32(rand_bits).reshape(mag.shape)
    saturate = mag >= 6.0
    denormal = (~saturate) & (mag < 1.0)
    low = denormal & (mag < 0.5)
    high = denormal & (~low)
    two33 = torch.tensor(float(2 ** 33 - 2), dtype=torch.float32)   # == 2^33 in fp32
    two32 = torch.tensor(float(2 ** 32 - 1), dtype=torch.float32)   # == 2^32 in fp32
    # lanes outside their range are masked below; clamp so the int64 cast is defined
    t_low = torch.where(low, mag * two33, torch.zeros_like(mag)).to(torch.int64)
    t_high = torch.where(high, (mag * 2 - 1) * two32, torch.zeros_like(mag)).to(torch.int64)
    den = torch.where(low, (r <= t_low).to(torch.int64), torch.zeros_like(r))
    den = torch.where(high, 1 + (r <= t_high).to(torch.int64), den)
    nor = (mag_bits + ((1 - 127) << 23) + (r & 0x3FFFFF)) & 0xFFFFFFFF
    nor = (nor >> 22) & 0xFF
    code = torch.full_like(mag_bits, 7)
    code = torch.where(saturate, code, torch.where(denormal, den, nor))
    code = code | (sign >> 28)
    return code.to(torch.uint8)


# --------------------------------------------------------------------------- decode / pack (Q3, Q6)
def decode_e2m1(code: torch.Tensor) -> torch.Tensor:
    """4-bit code (uint8, low nibble) -> fp32 value. triton_fp4_ops.py:111-132."""
    c = code.to(torch.int64)
    s = c & 0x8
    c = c ^ s
    bits = (((c >> 1) - 1 + 127) << 23) | ((c & 1) << 22)
    bits = torch.where(c == 0, torch.zeros_like(bits), bits)
    bits = torch.where(c == 1, torch.full_like(bits, 0x3F000000), bits)
    bits = bits | (s << 28)
    # values >= 2^31 need a wrap into int32 range
    bits = torch.where(bits >= 2 ** 31, bits - 2 ** 32, bits)
    return bits.to(torch.int32).view(torch.float32)


def pack_nibbles(codes: torch.Tensor) -> torch.Tensor:
    """[..., C] codes -> [..., C/2] bytes; even element in the low nibble. mxfp_quantization.py:115,186."""
    c = codes.contiguous()
    return (c[..., 0::2] | (c[..., 1::2] << 4)).contiguous()


def unpack_nibbles(packed: torch.Tensor) -> torch.Tensor:
    lo = packed & 0xF
    hi = packed >> 4
    return torch.stack([lo, hi], dim=-1).reshape(*packed.shape[:-1], packed.shape[-1] * 2)


def _scale_fp32(scales: torch.Tensor) -> torch.Tensor:
    """uint8 E8M0 -> fp32 2^(s-127), built by shifting into the exponent field (mxfp_quantization.py:117)."""
    return (scales.to(torch.int32) << 23).view(torch.float32)


def _expand_scales(s_fp: torch.Tensor, R: int, C: int, is_2d_block: bool) -> torch.Tensor:
    if is_2d_block:
        return s_fp.reshape(R // BLOCK, 1, C // BLOCK, 1).expand(R // BLOCK, BLOCK, C // BLOCK, BLOCK).reshape(R, C)
    return s_fp.reshape(R, C // BLOCK, 1).expand(R, C // BLOCK, BLOCK).reshape(R, C)


# --------------------------------------------------------------------------- quantize / dequantize (Q5, Q6)
def quantize(
    x: torch.Tensor,
    axis: int = -1,
    is_2d_block: bool = False,
    use_sr: bool = False,
    rand_bits: Optional[torch.Tensor] = None,
    clip_mode: str = "none",
    use_uos: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16/fp32 tensor -> (packed codes uint8, E8M0 scales uint8), layouts as the reference returns them.

    mxfp_quantization.py:410-484: the quantisation axis is moved last with a
    transpose view, leading dims are flattened, the results are reshaped and
    transposed back, so ``axis=0`` on ``[M, C]`` returns logical ``[M/2, C]``
    codes whose memory is ``[C][M/2]``.
    """
    assert x.dtype in (torch.bfloat16, torch.float32)
    if clip_mode not in ("none", "static", "dynamic"):
        raise ValueError(f"Invalid clip mode: {clip_mode}")
    assert x.shape[axis] % BLOCK == 0
    xt = x.transpose(axis, -1)
    shape = xt.shape
    x2 = xt.reshape(-1, shape[-1]).contiguous()
    R, C = x2.shape
    r2 = None
    if use_sr:
        assert rand_bits is not None and rand_bits.shape == x.shape
        rb = rand_bits
        if rb.dtype == torch.uint32:
            rb = rb.view(torch.int32)
        r2 = rb.transpose(axis, -1).reshape(-1, shape[-1]).contiguous()
    if is_2d_block:
        assert x.dim() >= 2 and shape[-2] % BLOCK == 0
        lead = int(math.prod(shape[:-2])) if len(shape) > 2 else 1
        xb = x2.reshape(lead, shape[-2], C)
        scales = torch.stack([block_scales(xb[i], True, clip_mode, use_uos) for i in range(lead)])
        s_full = torch.stack([_expand_scales(_scale_fp32(scales[i]), shape[-2], C, True) for i in range(lead)]).reshape(R, C)
        scales_shape = (*shape[:-2], shape[-2] // BLOCK, C // BLOCK)
    else:
        scales = block_scales(x2, False, clip_mode, use_uos)
        s_full = _expand_scales(_scale_fp32(scales), R, C, False)
        scales_shape = (*shape[:-1], C // BLOCK)
    xv = x2
    if clip_mode == "static":
        xv = x2 * (3.0 / 4.0)  # in the input dtype, mxfp_quantization.py:321-322
    q = xv.float() / s_full
    codes = encode_e2m1_sr(q, r2) if use_sr else encode_e2m1_rne(q)
    packed = pack_nibbles(codes).reshape(*shape[:-1], C // 2)
    scales = scales.reshape(scales_shape)
    return packed.transpose(axis, -1), scales.transpose(axis, -1)


def dequantize(
    codes: torch.Tensor,
    scales: torch.Tensor,
    output_dtype: torch.dtype = torch.float32,
    axis: int = -1,
    is_2d_block: bool = False,
    clip_mode: str = "none",
) -> torch.Tensor:
    """(packed codes, scales) -> tensor of ``output_dtype``. mxfp_quantization.py:487-545, triton_fp4_ops.py:98-134.

    value = fp32(grid value) * 2^(s-127) in fp32, optionally * 4/3 (static clip), cast once to the output dtype.
    """
    ct = codes.transpose(axis, -1)
    st = scales.transpose(axis, -1)
    shape = (*ct.shape[:-1], ct.shape[-1] * 2)
    c2 = ct.reshape(-1, ct.shape[-1]).contiguous()
    R, C = c2.shape[0], c2.shape[1] * 2
    vals = decode_e2m1(unpack_nibbles(c2))
    if is_2d_block:
        lead = int(math.prod(shape[:-2])) if len(shape) > 2 else 1
        sb = st.reshape(lead, shape[-2] // BLOCK, C // BLOCK)
        s_full = torch.stack([_expand_scales(_scale_fp32(sb[i].contiguous()), shape[-2], C, True) for i in range(lead)]).reshape(R, C)
    else:
        s_full = _expand_scales(_scale_fp32(st.reshape(R, C // BLOCK).contiguous()), R, C, False)
    y = vals * s_full
    if clip_mode == "static":
        y = y * (4.0 / 3.0)
    return y.to(output_dtype).reshape(shape).transpose(axis, -1)


# --------------------------------------------------------------------------- Hadamard (Q7)
def hadamard_matrix(signs: torch.Tensor, perm: Optional[torch.Tensor]) -> torch.Tensor:
    """The 32x32 fp32 matrix the reference multiplies with.

    hadamard.py:80-87,144-150: ``W0 = diag(Q) @ H`` with ``H[t, j] = (-1)^popcount(t & j)``
    (the butterfly in ``_matmul_hadU`` yields Sylvester order); transform.py:127-128:
    ``W = W0[perm][:, perm]``, i.e. ``W[i, j] = Q[perm[i]] * H[perm[i], perm[j]]``.
    """
    n = BLOCK
    idx = torch.arange(n)
    pc = torch.zeros(n, n, dtype=torch.int64)
    v = idx[:, None] & idx[None, :]
    for b in range(5):
        pc += (v >> b) & 1
    H = (1 - 2 * (pc & 1)).float()
    W0 = signs.float().reshape(n, 1) * H
    if perm is None:
        return W0
    p = perm.long()
    return W0[p][:, p]


def rht_left(x: torch.Tensor, signs: torch.Tensor, perm: Optional[torch.Tensor]) -> torch.Tensor:
    """Randomized Hadamard transform along dim 0 in blocks of 32 rows, FIXED summation order.

    transform.py:137-142 (``left_mul``): ``Y[32b+i, c] = cast(sum_j W[i, j] * fp32(X[32b+j, c]) / fp32(sqrt 32))``.
    The order of the 32-term fp32 sum is pinned here as follows (the HIP kernel
    does the same): scatter ``z[perm[j]] = fp32(X[32b+j])``; five in-place
    butterfly stages with strides h = 1, 2, 4, 8, 16, each ``(a, b) -> (a + b, a - b)``
    on index pairs ``(k, k + h)`` with ``k & h == 0``; then
    ``Y[32b+i] = cast((Q[perm[i]] * z[perm[i]]) / fp32(sqrt 32))``.
    """
    M, C = x.shape
    assert M % BLOCK == 0
    n = BLOCK
    p = torch.arange(n) if perm is None else perm.long()
    z = torch.empty(M // n, n, C, dtype=torch.float32)
    xb = x.float().reshape(M // n, n, C)
    z[:, p, :] = xb
    h = 1
    while h < n:
        zz = z.reshape(M // n, n // (2 * h), 2, h, C)
        a = zz[:, :, 0].clone()
        b = zz[:, :, 1].clone()
        zz[:, :, 0] = a + b
        zz[:, :, 1] = a - b
        h *= 2
    y = z[:, p, :] * signs.float()[p].reshape(1, n, 1)
    y = y / torch.tensor(SQRT32_F32, dtype=torch.float32)
    return y.reshape(M, C).to(x.dtype)


def rht(x: torch.Tensor, signs: torch.Tensor, perm: Optional[torch.Tensor], inverse: bool = False, left_mul: bool = False) -> torch.Tensor:
    """All four forms of ``HadamardTransform.__call__`` (transform.py:115-142), FIXED summation order.

    ``left_mul``: ``V @ x`` over the last two dims in blocks of 32 rows, else ``x @ V`` in blocks of 32 along the last
    dim (matrix.py:152-161 unflattens the larger operand), ``V = W`` or ``W.T`` (``inverse``, transform.py:130-131).
    With ``W[i, j] = Q[p[i]] H[p[i], p[j]]`` every form is: scatter the 32 inputs to ``z[p[j]]``, butterfly as in
    :func:`rht_left`, gather ``z[p[i]]``; ``Q`` multiplies the gathered outputs where the output index is W's row index
    (``W @ x`` and ``x @ W.T``) and the scattered inputs where the input index is (``W.T @ x`` and ``x @ W``).
    """
    if not left_mul:
        return rht(x.transpose(-1, -2) if x.dim() >= 2 else x.reshape(-1, 1), signs, perm, not inverse, True).transpose(-1, -2).reshape(x.shape)
    shape = x.shape
    M, C = shape[-2], shape[-1]
    assert M % BLOCK == 0
    n = BLOCK
    p = torch.arange(n) if perm is None else perm.long()
    q = signs.float()[p].reshape(1, n, 1)
    xb = x.float().reshape(-1, n, C)
    z = torch.empty_like(xb)
    z[:, p, :] = xb * q if inverse else xb
    h = 1
    while h < n:
        zz = z.reshape(z.shape[0], n // (2 * h), 2, h, C)
        a = zz[:, :, 0].clone()
        b = zz[:, :, 1].clone()
        zz[:, :, 0] = a + b
        zz[:, :, 1] = a - b
        h *= 2
    y = z[:, p, :]
    if not inverse:
        y = y * q
    y = y / torch.tensor(SQRT32_F32, dtype=torch.float32)
    return y.reshape(shape).to(x.dtype)


def rht_dense(x: torch.Tensor, signs: torch.Tensor, perm: Optional[torch.Tensor], inverse: bool = False, left_mul: bool = False,
              dtype=torch.float32) -> torch.Tensor:
    """The reference's own formulation (transform.py:125-142 with matrix.py:152-161): dense matmuls, the backend's order."""
    W = hadamard_matrix(signs, perm).to(dtype)
    if inverse:
        W = W.T
    v = x.to(dtype)
    if left_mul:
        y = (W @ v.unflatten(-2, (v.shape[-2] // BLOCK, BLOCK))).flatten(-3, -2)
    else:
        y = (v.unflatten(-1, (v.shape[-1] // BLOCK, BLOCK)) @ W).flatten(-2, -1)
    return y / torch.tensor(SQRT32_F32, dtype=torch.float32).to(dtype)


def rht_left_dense(x: torch.Tensor, signs: torch.Tensor, perm: Optional[torch.Tensor], dtype=torch.float32) -> torch.Tensor:
    """Same transform as a dense block-diagonal matmul (the reference's formulation); summation order is the backend's."""
    M, C = x.shape
    W = hadamard_matrix(signs, perm).to(dtype)
    y = W @ x.to(dtype).reshape(M // BLOCK, BLOCK, C)
    y = y / torch.tensor(SQRT32_F32, dtype=torch.float32).to(dtype)
    return y.reshape(M, C)


# --------------------------------------------------------------------------- GEMM (Q9)
def _dq_operand(codes, scales, packed_along_k: bool, operand_is_kxn: bool, is_2d: bool, dtype):
    """Decode one GEMM operand to a dense [rows, K] (A-like) or [K, N] matrix following blockwise_mxfp4_gemm's flags."""
    # logical tensor dims: codes [d0, d1] with the packed dim halved
    if packed_along_k == (not operand_is_kxn):
        # packed along the last dim
        return dequantize(codes, scales, dtype, axis=-1, is_2d_block=is_2d)
    return dequantize(codes, scales, dtype, axis=0, is_2d_block=is_2d)


def gemm_ref(a, a_s, b, b_s, use_2dblock_a=False, use_2dblock_b=False, k_pack_a=True, k_pack_b=True,
             trans_a=False, trans_b=False, dtype=torch.float64) -> torch.Tensor:
    """matmul of the dequantized operands, flags as blockwise_mxfp4_gemm (mxfp_linear.py:142-255).

    a: [M, K] (or [K, M] if trans_a) with the packed dim halved; packed along K when k_pack_a.
    b: [K, N] (or [N, K] if trans_b); packed along K when k_pack_b.
    Scales index [row, K/32] / [K/32, row] (1D) or [rows/32, K/32] (2D) in the same orientation as the codes.
    """
    # A: K is dim 1 unless trans_a
    a_k_is_last = not trans_a
    a_axis = -1 if (k_pack_a == a_k_is_last) else 0
    a_dq = dequantize(a, a_s, torch.float32, axis=a_axis, is_2d_block=use_2dblock_a).to(dtype)
    b_k_is_last = trans_b
    b_axis = -1 if (k_pack_b == b_k_is_last) else 0
    b_dq = dequantize(b, b_s, torch.float32, axis=b_axis, is_2d_block=use_2dblock_b).to(dtype)
    A = a_dq.T if trans_a else a_dq
    B = b_dq.T if trans_b else b_dq
    return A @ B


def rel_frobenius(got: torch.Tensor, ref: torch.Tensor) -> float:
    g = got.double()
    r = ref.double()
    return float((g - r).norm() / r.norm().clamp_min(1e-300))


# --------------------------------------------------------------------------- linear (Q8)
def linear_forward_ref(x, w, use_2dblock_x=False, use_2dblock_w=True, hadamard=None, clip_mode="none", dtype=torch.float64, use_uos=False):
    """Forward of MXFP4LinearFunction (mxfp_linear.py:265-422) on its dequantize-and-matmul branch.

    Returns (y, saved) where saved holds the operands backward needs:
    the token-axis (axis 0) quantisation of H.x and the weight codes/scales.
    """
    x2 = x.reshape(-1, x.shape[-1])
    xq, xs = quantize(x2, axis=-1, is_2d_block=use_2dblock_x, use_uos=use_uos)
    wq, ws = quantize(w, axis=-1, is_2d_block=use_2dblock_w, use_uos=use_uos)
    y = gemm_ref(xq, xs, wq, ws, use_2dblock_x, use_2dblock_w, trans_b=True, dtype=dtype)
    saved = {}
    if not use_2dblock_w:
        wq, ws = quantize(w, axis=0, is_2d_block=False, use_uos=use_uos)
    if not use_2dblock_x:
        xh = rht_left(x2, *hadamard) if hadamard is not None else x2
        xq, xs = quantize(xh, axis=0, is_2d_block=False, clip_mode=clip_mode, use_uos=use_uos)
    saved.update(x_q=xq, x_s=xs, w_q=wq, w_s=ws)
    return y, saved


def linear_backward_ref(grad_out, saved, use_2dblock_x=False, use_2dblock_w=True, use_sr_grad=False, rand_bits=None,
                        hadamard=None, clip_mode="none", dtype=torch.float64, use_uos=False):
    """Backward of MXFP4LinearFunction (mxfp_linear.py:424-570): returns (dX, dW) in ``dtype``."""
    g2 = grad_out.reshape(-1, grad_out.shape[-1])
    if use_2dblock_x:
        gq, gs = quantize(g2, axis=-1, is_2d_block=True, use_sr=use_sr_grad, rand_bits=rand_bits, use_uos=use_uos)
        gq_m, gs_m = gq, gs
    else:
        gq, gs = quantize(g2, axis=-1, is_2d_block=False, use_sr=use_sr_grad, rand_bits=rand_bits, use_uos=use_uos)
        gh = rht_left(g2, *hadamard) if hadamard is not None else g2
        gq_m, gs_m = quantize(gh, axis=0, is_2d_block=False, use_sr=use_sr_grad, rand_bits=rand_bits, clip_mode=clip_mode, use_uos=use_uos)
    dx = gemm_ref(gq, gs, saved["w_q"], saved["w_s"], use_2dblock_x, use_2dblock_w, k_pack_b=not use_2dblock_w, dtype=dtype)
    dw = gemm_ref(gq_m, gs_m, saved["x_q"], saved["x_s"], use_2dblock_x, use_2dblock_x, trans_a=True,
                  k_pack_a=not use_2dblock_x, k_pack_b=not use_2dblock_x, dtype=dtype)
    if clip_mode == "static":
        dw = dw * (16.0 / 9.0)
    return dx, dw


# --------------------------------------------------------------------------- differentiable gradient estimator
E2M1_BREAK_POINTS = (-6, -4, -3, -2, -1.5, -1, -0.5, 0, 0.5, 1, 1.5, 2, 3, 4, 6)


def dge_bwd_ref(x: torch.Tensor, k: float = 5.0) -> torch.Tensor:
    """Multiplier of the weight gradient at the quantised weight's grid values ``x`` (fp32), alto/kernels/dge/dge.py:80-93
    for float4_e2m1fn_x2 (break points :46): the interval that holds x (searchsorted from the left, minus one, clamped),
    its half width and mid point, then clamp(half^(1-1/k) |x - mid|^(1/k-1) / k, 0, 3)."""
    bp = torch.tensor(E2M1_BREAK_POINTS, dtype=torch.float32)
    xc = x.float().contiguous()
    idx = torch.searchsorted(bp, xc, right=False) - 1
    idx = idx.clamp(0, len(bp) - 2)
    half = (bp[idx + 1] - bp[idx]) / 2.0
    mid = bp[idx] + half
    return torch.clamp(half ** (1 - 1 / k) * (xc - mid).abs() ** (1 / k - 1) / k, 0, 3.0)


def weight_grid_values(w_q: torch.Tensor, axis: int = -1) -> torch.Tensor:
    """E2M1 grid values of packed weight codes, i.e. the dequantisation with unit scales that mxfp_linear.py:549-566 feeds
    to dge_bwd."""
    ct = w_q.transpose(axis, -1)
    vals = decode_e2m1(unpack_nibbles(ct.reshape(-1, ct.shape[-1]).contiguous()))
    return vals.reshape(*ct.shape[:-1], ct.shape[-1] * 2).transpose(axis, -1)


# --------------------------------------------------------------------------- grouped (Q10)
def indices_from_offsets(offs: torch.Tensor) -> torch.Tensor:
    """Cumulative group ends -> per-row expert id. dsgemm_utils.py:96-112 (bucketize(arange(offs[-1]), offs, right=True))."""
    total = int(offs[-1])
    return torch.bucketize(torch.arange(total, dtype=torch.int32), offs.to(torch.int32), right=True, out_int32=True)


def grouped_gemm_ref(a_q, a_s, w_q, w_s, expert_indices, use_2dblock_x=False, use_2dblock_w=True, trans_weights=True,
                     dtype=torch.float64) -> torch.Tensor:
    """out[r] = dq(A)[r] @ dq(W[e(r)])^T (cg_forward.py:200-303); rows beyond len(expert_indices) stay 0.

    w_q: [E, N, K/2] if trans_weights else [E, K/2, N] (packed along K either way).
    """
    a = dequantize(a_q, a_s, torch.float32, axis=-1, is_2d_block=use_2dblock_x).to(dtype)
    E = w_q.shape[0]
    w_axis = -1 if trans_weights else -2
    w = dequantize(w_q, w_s, torch.float32, axis=w_axis, is_2d_block=use_2dblock_w).to(dtype)
    if not trans_weights:
        w = w.transpose(-1, -2)  # -> [E, N, K]
    out = torch.zeros(a.shape[0], w.shape[1], dtype=dtype)
    idx = expert_indices.long()
    for e in range(E):
        rows = (idx == e).nonzero().flatten()
        if rows.numel():
            out[rows] = a[rows] @ w[e].T
    return out


def grouped_gemm_dx_ref(go_q, go_s, w_q, w_s, expert_indices, use_2dblock_x=False, use_2dblock_w=True, trans_weights=True,
                        k_pack_w=False, dtype=torch.float64) -> torch.Tensor:
    """dX[r] = dq(dY)[r] @ dq(W[e(r)]) (cg_backward.py:500-593). Reduction over N; W packed along N iff k_pack_w."""
    go = dequantize(go_q, go_s, torch.float32, axis=-1, is_2d_block=use_2dblock_x).to(dtype)
    E = w_q.shape[0]
    # weights are [E, N, K] (trans_weights) or [E, K, N]; packed along N when k_pack_w else along K
    n_axis = -2 if trans_weights else -1
    k_axis = -1 if trans_weights else -2
    w = dequantize(w_q, w_s, torch.float32, axis=n_axis if k_pack_w else k_axis, is_2d_block=use_2dblock_w).to(dtype)
    if not trans_weights:
        w = w.transpose(-1, -2)  # [E, N, K]
    out = torch.zeros(go.shape[0], w.shape[2], dtype=dtype)
    idx = expert_indices.long()
    for e in range(E):
        rows = (idx == e).nonzero().flatten()
        if rows.numel():
            out[rows] = go[rows] @ w[e]
    return out


def grouped_gemm_dw_ref(go_q, go_s, x_q, x_s, expert_indices, num_experts, use_2dblock_x=False, trans_weights=True,
                        dtype=torch.float64) -> torch.Tensor:
    """dW[e] = sum_{rows of e} dq(dY)^T @ dq(X) (cg_backward.py:398-497); operands packed along tokens unless 2D."""
    axis = -1 if use_2dblock_x else 0
    go = dequantize(go_q, go_s, torch.float32, axis=axis, is_2d_block=use_2dblock_x).to(dtype)
    x = dequantize(x_q, x_s, torch.float32, axis=axis, is_2d_block=use_2dblock_x).to(dtype)
    N, K = go.shape[1], x.shape[1]
    out = torch.zeros(num_experts, N, K, dtype=dtype)
    idx = expert_indices.long()
    for e in range(num_experts):
        rows = (idx == e).nonzero().flatten()
        if rows.numel():
            out[e] = go[rows].T @ x[rows]
    return out if trans_weights else out.transpose(-1, -2)
