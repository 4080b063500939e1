"""CPU oracle for the quantized-matmul operators (TEST INFRASTRUCTURE ONLY).

This module restates, in numpy, the arithmetic that the reference operator
definitions prescribe.  It is the *checker* for the HIP kernels: only tests,
the smoke check and the benchmark's cpu-baseline leg may import it.  The
product package never does.

Every function cites the reference file:line it follows (paths relative to
the reference checkout).

Pinning status of each function (what independent evidence fixes it):

  round_half_away          closed form; tie cases; equals C roundf (checked against the C restatement)
  symmetric_quantize       invariants (scale == amax/qmax bit-for-bit, max|q| == qmax, odd symmetry),
                           constructed ties, brute force over all f16 patterns against the reference's own half
                           type (oracle/_ref where built, and its recorded outputs in tests/golden/ref_half_vectors.npz),
                           reference test shapes
  reference_cpu_quant_matmul  bit for bit against the reference's half type (oracle/_ref and the golden vectors)
  symmetric_dequantize     closed form (one multiply); round trip at the reference's tolerance
  symmetric_quant_matmul   reduces to a library matmul on the dequantized weights; exact small-integer cases
  quant_matmul_split_k     sum over parts == full; zero-padded tail part
  resolve_k_parts          direct evaluation of the reference's formula table
  e4m3_decode / e4m3_encode  exhaustive over 256 codes against torch.float8_e4m3fn; reference KAT literals
  matmul_f8 / _scaled      integer-valued inputs -> exact int64 result (the reference's own test recipe)
  fp8_quantize_per_tensor, group_quantize_int4, pack/unpack_int4, w4a16_matmul, fp8_matmul_per_tensor
                           defined by the benchmark configuration, not by a reference function:
                           PARITY UNPINNED by any reference test (closed forms / round trips only)
"""
from __future__ import annotations

from typing import Sequence, Tuple, Union

import numpy as np

# --------------------------------------------------------------------------------------
# dtype helpers.  numpy has no bfloat16: bf16 tensors are carried as float32 arrays whose
# values are bf16-representable, and every bf16 operation is "float32 op, then round".
# --------------------------------------------------------------------------------------

INT_MAX = {'int8': 127, 'int16': 32767, 'int4b': 7}  # ir/dtypes/integer.py:77-78, integer_subbyte.py:49
INT_NP = {'int8': np.int8, 'int16': np.int16}


def to_bf16(x: np.ndarray) -> np.ndarray:
    """Round float32 values to the nearest bfloat16 (ties to even); result kept as float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32).copy()
    nan = np.isnan(x)
    if nan.any():
        out[nan] = np.float32(np.nan)
    return out.reshape(x.shape)


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """uint16 bit patterns of bf16-representable float32 values."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return (x.view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(b: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def _round_to(x32: np.ndarray, dtype: str) -> np.ndarray:
    """Round a float32 result to `dtype`, returned in that dtype's carrier array type."""
    if dtype == 'float32':
        return x32.astype(np.float32)
    if dtype == 'float16':
        return x32.astype(np.float16)
    if dtype == 'bfloat16':
        return to_bf16(x32)
    raise ValueError(dtype)


def _dtype_of(x: np.ndarray, dtype: Union[str, None]) -> str:
    if dtype is not None:
        return dtype
    if x.dtype == np.float16:
        return 'float16'
    if x.dtype == np.float32:
        return 'float32'
    raise ValueError('unsupported array dtype {}'.format(x.dtype))


def round_half_away(x: np.ndarray) -> np.ndarray:
    """roundf semantics: nearest integer, ties away from zero.

    The reference lowers `round` to `roundf`/`std::round` for float32 on every target
    (ir/primitives/cpu/math/float32.py:40) and to std::round(float) for the CPU half and
    bfloat16 types (include/hidet/runtime/cpu/float16.h:747-750).  numpy's `round` is
    ties-to-even, so the rounding is spelled out: for |x| < 2**23 the fraction x - trunc(x)
    is exact in float32.
    """
    x = np.asarray(x, dtype=np.float32)
    t = np.trunc(x)
    frac = np.abs(x - t)
    return (t + np.sign(x) * (frac >= np.float32(0.5))).astype(np.float32)


# --------------------------------------------------------------------------------------
# symmetric quantize / dequantize
# --------------------------------------------------------------------------------------

def _normalize_dims(dims: Union[int, Sequence[int]], rank: int) -> Tuple[int, ...]:
    if isinstance(dims, int):
        dims = [dims]
    out = []
    for d in dims:
        if d < 0:
            d += rank
        if not 0 <= d < rank:
            raise ValueError('dim out of range')
        out.append(d)
    return tuple(sorted(set(out)))


def symmetric_quantize(w: np.ndarray, quant_type: str = 'int8', dims: Union[int, Sequence[int]] = -1,
                       dtype: Union[str, None] = None, target: str = 'cpu') -> Tuple[np.ndarray, np.ndarray]:
    """(wq, scale) of graph/ops/quant/symmetric.py:23-47,82-84.

    `target` selects the reference's lowering of `round`, which depends on where the operator runs: 'cpu' rounds
    ties away from zero for every dtype (roundf; include/hidet/runtime/cpu/float16.h:747-750, bfloat16.h:522-524),
    'gpu' rounds ties away for float32 (ir/primitives/hip/math/float32.py:40) and ties to even for float16 and
    bfloat16 (hrint: ir/primitives/hip/math/float16.py:42, cuda/math/float16.py:73, cuda/math/bfloat16.py:29). The HIP
    kernels follow 'gpu'; the vectors recorded from the reference's CPU half type pin 'cpu'.

    `dims` are the reduced axes; `scale` has the remaining axes' shape.  All arithmetic is
    evaluated in the dtype of `w` (ir/dtypes/promotion.py:128-148): for float16/bfloat16 each of
    `amax / qmax` and `w / scale` is a float32 operation rounded back to the narrow type
    (include/hidet/runtime/cpu/float16.h:441-444), then `round` (ties away) and an integer cast.
    The reference has no clamp: |w / scale| <= qmax by construction in float32 and float16.  In
    bfloat16 the twice-rounded quotient of the amax element can reach qmax + 0.5, which rounds
    to qmax + 1 and overflows the integer cast (undefined in the reference; the same happens in
    float16 when the scale is subnormal).  The cast saturates to the integer type's range
    [-qmax - 1, qmax] here and in the kernels, which changes nothing wherever the reference is
    defined.

    A slice whose amax is 0 has scale 0 and the reference evaluates 0/0 (undefined integer
    cast).  Defined here, and in the kernels, as scale = 0 and code = 0.
    """
    dt = _dtype_of(w, dtype)
    qmax = np.float32(INT_MAX[quant_type])
    red = _normalize_dims(dims, w.ndim)
    w32 = np.asarray(w, dtype=np.float32)
    amax = np.max(np.abs(w32), axis=red, keepdims=True, initial=0)  # exact in any order; empty slice -> 0
    scale32 = _round_to(amax / qmax, dt).astype(np.float32)  # one division, rounded to w's dtype
    with np.errstate(divide='ignore', invalid='ignore'):
        quot = _round_to(w32 / scale32, dt).astype(np.float32)  # one division, rounded to w's dtype
    quot = np.where(scale32 == 0, np.float32(0), quot)
    if target not in ('cpu', 'gpu'):
        raise ValueError("target must be 'cpu' or 'gpu', got {!r}".format(target))
    rounded = np.rint(quot) if (target == 'gpu' and dt != 'float32') else round_half_away(quot)
    q = np.clip(rounded, -qmax - 1, qmax).astype(INT_NP[quant_type])
    scale = _round_to(np.squeeze(scale32, axis=red), dt)
    return q, scale


def symmetric_dequantize(wq: np.ndarray, scale: np.ndarray, dims: Union[int, Sequence[int]] = -1,
                         dtype: Union[str, None] = None) -> np.ndarray:
    """w = cast(wq, scale.dtype) * scale  (graph/ops/quant/symmetric.py:50-61): one multiply,
    rounded to the scale's dtype."""
    dt = _dtype_of(scale, dtype)
    red = _normalize_dims(dims, wq.ndim)
    s32 = np.expand_dims(np.asarray(scale, dtype=np.float32), axis=red)
    return _round_to(wq.astype(np.float32) * s32, dt)


# --------------------------------------------------------------------------------------
# W8A16 matmul
# --------------------------------------------------------------------------------------

def symmetric_quant_matmul(a: np.ndarray, weight: np.ndarray, scale: np.ndarray, acc: str = 'f32') -> np.ndarray:
    """c[..., m, n] = sum_k a[..., m, k] * (f16(weight[k, n]) * scale[n])   (graph/ops/quant/matmul.py:57-72).

    The dequantized weight is rounded to float16 before it meets `a` (definition order); the
    sum is accumulated in float32 (or float64 with acc='f64') and the result rounded to float16.
    This is the parity target for every W8A16 kernel.
    """
    if a.dtype != np.float16 or weight.dtype != np.int8:
        raise ValueError('expect float16 a and int8 weight')
    if weight.ndim != 2 or a.ndim < 2 or a.shape[-1] != weight.shape[0] or scale.shape[0] != weight.shape[1]:
        raise ValueError('shape mismatch')
    wd = symmetric_dequantize(weight, scale.astype(np.float16), dims=0)  # [K, N] float16
    t = np.float64 if acc == 'f64' else np.float32
    c = np.matmul(a.astype(t), wd.astype(t))
    return c.astype(np.float32).astype(np.float16)


def quant_matmul_split_k(a: np.ndarray, weight: np.ndarray, scale: np.ndarray, parallel_k_parts: int) -> np.ndarray:
    """Output [k_parts, ..., M, N] of graph/ops/quant/matmul_f16_i8.py:60-86: part p sums
    k in [p*ceil(K/parts), (p+1)*ceil(K/parts)) with out-of-range k contributing zero."""
    k_size = a.shape[-1]
    ext = -(-k_size // parallel_k_parts)
    parts = []
    for p in range(parallel_k_parts):
        lo, hi = min(p * ext, k_size), min((p + 1) * ext, k_size)
        if hi > lo:
            parts.append(symmetric_quant_matmul(np.ascontiguousarray(a[..., lo:hi]), weight[lo:hi], scale))
        else:
            parts.append(np.zeros(a.shape[:-1] + (weight.shape[1],), dtype=np.float16))
    return np.stack(parts, axis=0)


def reference_cpu_quant_matmul(a: np.ndarray, weight: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """What the reference's CPU route computes for a 2-D `a`: one output element per loop
    iteration, serial k, every multiply and add rounded to float16, float16 accumulator
    (ir/schedulers/base.py:347-371 takes the accumulator dtype from the value;
    include/hidet/runtime/cpu/float16.h:424-444).  Pure numpy over k; small shapes only."""
    m, k = a.shape
    n = weight.shape[1]
    s = scale.astype(np.float16).astype(np.float32)
    a32 = a.astype(np.float32)
    accum = np.zeros((m, n), dtype=np.float32)  # holds float16-representable values
    for kk in range(k):
        wd = (weight[kk].astype(np.float32) * s).astype(np.float16).astype(np.float32)  # [n]
        prod = (a32[:, kk:kk + 1] * wd[None, :]).astype(np.float16).astype(np.float32)
        accum = (accum + prod).astype(np.float16).astype(np.float32)
    return accum.astype(np.float16)


def resolve_k_parts(parallel_k: Union[str, int], batch: int, m: int, n: int, k: int,
                    concurrent_blocks: int = 80 * 5) -> int:
    """k_parts policy of graph/ops/quant/resolve.py:37-96 ('search' is a timing loop, not a formula)."""
    cdiv = lambda x, y: -(-x // y)
    if isinstance(parallel_k, str):
        if parallel_k == 'default':
            blocks = batch * cdiv(m, 64) * cdiv(n, 64)
            return min(cdiv(concurrent_blocks, blocks), cdiv(k, 64))
        if parallel_k == 'disabled':
            return 1
        raise ValueError('invalid parallel_k: {}'.format(parallel_k))
    if isinstance(parallel_k, int):
        return min(max(parallel_k, 1), 32)
    raise ValueError('invalid parallel_k: {}'.format(parallel_k))


# --------------------------------------------------------------------------------------
# group-wise int4 (benchmark-defined; PARITY UNPINNED by reference tests)
# --------------------------------------------------------------------------------------

def pack_int4(q: np.ndarray) -> np.ndarray:
    """Two signed 4-bit codes per byte along the innermost axis, low nibble first: flattened
    element o lives in byte o//2 at bit (o%2)*4 (transforms/lower_integer_subbyte.py:103-113)."""
    if q.shape[-1] % 2:
        raise ValueError('innermost extent must be even')
    u = (q.astype(np.int16) & 0xF).astype(np.uint8)
    return (u[..., 0::2] | (u[..., 1::2] << 4)).astype(np.uint8)


def unpack_int4(p: np.ndarray) -> np.ndarray:
    """Inverse of pack_int4 with sign extension by shifts (lower_integer_subbyte.py:252-253)."""
    lo = ((p.astype(np.int8) << 4).astype(np.int8) >> 4).astype(np.int8)
    hi = (p.astype(np.int8) >> 4).astype(np.int8)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.int8)
    out[..., 0::2] = lo
    out[..., 1::2] = hi
    return out


def group_quantize_int4(w: np.ndarray, group_size: int = 128, scale_dtype: str = 'bfloat16'):
    """Symmetric signed-int4 quantization of w[K, N] with one scale per (k // group_size, n).

    The symmetric rule of symmetric.py:32-41 applied per group with qmax = 7: scale = amax / 7
    and code = round(w / scale) in float32 (w's dtype), codes clamped to [-7, 7]; the stored
    scale is that float32 scale rounded to `scale_dtype`.  Returns (packed uint8 [K, N/2],
    scales [K/g, N] as float32 carrier (bf16) or float16, codes int8 [K, N]).
    """
    k, n = w.shape
    if k % group_size:
        raise ValueError('K must be a multiple of the group size')
    w32 = np.asarray(w, dtype=np.float32).reshape(k // group_size, group_size, n)
    amax = np.max(np.abs(w32), axis=1, keepdims=True)
    scale32 = (amax / np.float32(7)).astype(np.float32)
    with np.errstate(divide='ignore', invalid='ignore'):
        quot = (w32 / scale32).astype(np.float32)
    quot = np.where(scale32 == 0, np.float32(0), quot)
    q = np.clip(round_half_away(quot), -7, 7).astype(np.int8).reshape(k, n)
    scales = _round_to(scale32[:, 0, :], scale_dtype)
    return pack_int4(q), scales, q


def w4a16_matmul(a: np.ndarray, packed: np.ndarray, scales: np.ndarray, group_size: int = 128,
                 dtype: str = 'bfloat16', acc: str = 'f32') -> np.ndarray:
    """c = a @ dequant(packed, scales): the dequantized weight is `dtype(q) * scale` rounded to
    `dtype` (the definition order of quant/matmul.py:63-70 carried over to groups), fp32 (or
    fp64) accumulation, result rounded to `dtype`.  `a` and `scales` are carriers of `dtype`."""
    q = unpack_int4(packed).astype(np.float32)
    s = np.repeat(np.asarray(scales, dtype=np.float32), group_size, axis=0)
    wd = _round_to(q * s, dtype).astype(np.float32)
    t = np.float64 if acc == 'f64' else np.float32
    c = np.matmul(np.asarray(a, dtype=np.float32).astype(t), wd.astype(t)).astype(np.float32)
    return _round_to(c, dtype)


# --------------------------------------------------------------------------------------
# FP8 e4m3fn (OCP): bias 7, max 448 (0x7E), 0x7F/0xFF NaN, no infinities, subnormals to 2**-9
# (ir/dtypes/floats.py:108-110)
# --------------------------------------------------------------------------------------

def e4m3_decode(code: np.ndarray) -> np.ndarray:
    c = np.asarray(code, dtype=np.uint8).astype(np.int32)
    sign = np.where(c & 0x80, np.float32(-1), np.float32(1))
    e = (c >> 3) & 0xF
    m = (c & 7).astype(np.float32)
    normal = np.ldexp(np.float32(1) + m / np.float32(8), e - 7)
    sub = np.ldexp(m / np.float32(8), -6)
    v = np.where(e == 0, sub, normal).astype(np.float32)
    v = np.where((c & 0x7F) == 0x7F, np.float32(np.nan), v)
    return (sign * v).astype(np.float32)


_E4M3_POS = None


def _e4m3_pos_table():
    global _E4M3_POS
    if _E4M3_POS is None:
        _E4M3_POS = e4m3_decode(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float64)  # 0 .. 448, increasing
    return _E4M3_POS


def e4m3_encode(x: np.ndarray) -> np.ndarray:
    """float32 -> e4m3fn code, round to nearest even, saturating to +-448 (NaN -> 0x7F | sign).

    Done by search in the table of the 127 non-negative finite values, so it shares no code
    with e4m3_decode's inverse formula beyond the table itself."""
    x = np.asarray(x, dtype=np.float32)
    tab = _e4m3_pos_table()
    ax = np.minimum(np.abs(x.astype(np.float64)), 448.0)
    hi = np.searchsorted(tab, ax, side='left')  # first index with tab[idx] >= ax
    hi = np.clip(hi, 0, len(tab) - 1)
    lo = np.clip(hi - 1, 0, len(tab) - 1)
    d_hi = tab[hi] - ax
    d_lo = ax - tab[lo]
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & ((lo & 1) == 0))  # tie: even mantissa == even code
    idx = np.where(pick_lo, lo, hi).astype(np.uint8)
    idx = np.where(np.isnan(x), np.uint8(0x7F), idx)
    sign = (np.signbit(x).astype(np.uint8) << 7).astype(np.uint8)
    return (idx | sign).astype(np.uint8)


# --------------------------------------------------------------------------------------
# FP8 e5m2 (OCP): bias 15, max 57344 (0x7B), 0x7C infinity, 0x7D-0x7F NaN, subnormals to 2**-16. A code is
# the upper byte of the float16 with the same value. Conversion from float32 rounds to nearest even and
# saturates finite values AND infinities to +-57344, NaN -> 0x7F: the saturate-to-finite conversion of the
# reference's float8_e5m2 type (include/hidet/runtime/cuda/float8_e5m2.h:6).
# --------------------------------------------------------------------------------------

def e5m2_decode(code: np.ndarray) -> np.ndarray:
    c = np.asarray(code, dtype=np.uint8).astype(np.uint16)
    return (c << np.uint16(8)).astype(np.uint16).view(np.float16).astype(np.float32)


_E5M2_POS = None


def _e5m2_pos_table() -> np.ndarray:
    global _E5M2_POS
    if _E5M2_POS is None:
        _E5M2_POS = e5m2_decode(np.arange(0x7C, dtype=np.uint8)).astype(np.float64)  # 0 .. 57344, ascending
    return _E5M2_POS


def e5m2_encode(x: np.ndarray) -> np.ndarray:
    """float32 -> e5m2 code by search in the table of the 124 non-negative finite values (ties to the even code)."""
    x = np.asarray(x, dtype=np.float32)
    tab = _e5m2_pos_table()
    ax = np.minimum(np.abs(x.astype(np.float64)), 57344.0)
    ax = np.where(np.isnan(ax), 0.0, ax)
    hi = np.clip(np.searchsorted(tab, ax, side='left'), 0, len(tab) - 1)
    lo = np.clip(hi - 1, 0, len(tab) - 1)
    d_hi, d_lo = tab[hi] - ax, ax - tab[lo]
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & ((lo & 1) == 0))
    idx = np.where(pick_lo, lo, hi).astype(np.uint8)
    idx = np.where(np.isnan(x), np.uint8(0x7F), idx)
    sign = (np.signbit(x).astype(np.uint8) << 7).astype(np.uint8)
    return (idx | sign).astype(np.uint8)


def fp8_quantize_per_tensor(x: np.ndarray) -> Tuple[np.ndarray, np.float32]:
    """scale = amax / 448 (float32), code = e4m3(x / scale)  (benchmark-defined)."""
    x = np.asarray(x, dtype=np.float32)
    scale = np.float32(np.max(np.abs(x), initial=0) / np.float32(448))
    if scale == 0:
        return np.zeros(x.shape, dtype=np.uint8), scale
    return e4m3_encode((x / scale).astype(np.float32)), scale


def _cast_out(c32: np.ndarray, out_dtype: str) -> np.ndarray:
    if out_dtype == 'float8_e4m3':
        return e4m3_encode(c32)
    if out_dtype == 'float8_e5m2':
        return e5m2_encode(c32)
    return _round_to(c32, out_dtype)


def matmul_f8(a_code: np.ndarray, b_code: np.ndarray, out_dtype: Union[str, None] = None, acc: str = 'f32',
              in_dtype: str = 'float8_e4m3') -> np.ndarray:
    """C[..., M, N] = cast(sum_k f32(A[..., M, k]) * f32(B[..., N, k])); A is [M, K] and B is
    [N, K], both K-major and both of `in_dtype`, float8_e4m3 or float8_e5m2 (graph/ops/matmul/matmul_f8.py:132-149,
    693-742).  The default output dtype is the input fp8 type (:714-715)."""
    t = np.float64 if acc == 'f64' else np.float32
    decode = e5m2_decode if in_dtype == 'float8_e5m2' else e4m3_decode
    out_dtype = in_dtype if out_dtype is None else out_dtype
    a = decode(a_code).astype(t)
    b = decode(b_code).astype(t)
    c = np.matmul(a, np.swapaxes(b, -1, -2)).astype(np.float32)
    return _cast_out(c, out_dtype)


def matmul_f8_scaled(a_code, b_code, scale_a, scale_b, out_dtype: str = 'bfloat16', block: int = 128,
                     in_dtype: str = 'float8_e4m3') -> np.ndarray:
    """Per K-block of 128: C += (sum_{k in blk} A*B) * scale_a[kb, m] * scale_b[nb, kb]
    (matmul_f8.py:357-363, 632-636); scale_a is [K/128, M], scale_b is [N/128, K/128]. Both operands are of
    `in_dtype`, float8_e4m3 or float8_e5m2 (the task asserts only that they agree, :386-389; _matmul_f8 admits both
    formats for the scaled form as well, :709-712)."""
    decode = e5m2_decode if in_dtype == 'float8_e5m2' else e4m3_decode
    a = decode(a_code)
    b = decode(b_code)
    m, k = a.shape
    n = b.shape[0]
    c = np.zeros((m, n), dtype=np.float32)
    for kb in range(k // block):
        part = np.matmul(a[:, kb * block:(kb + 1) * block], b[:, kb * block:(kb + 1) * block].T).astype(np.float32)
        sb = np.repeat(np.asarray(scale_b, dtype=np.float32)[:, kb], n // scale_b.shape[0])  # [N]
        c += part * np.asarray(scale_a, dtype=np.float32)[kb][:, None] * sb[None, :]
    return _cast_out(c, out_dtype)


def fp8_matmul_per_tensor(a_code, b_code, scale_a, scale_b, out_dtype: str = 'bfloat16', acc: str = 'f32'):
    """out = cast((sum_k f32(Aq) f32(Bq)) * (sa * sb))  (benchmark-defined per-tensor scaling)."""
    t = np.float64 if acc == 'f64' else np.float32
    a = e4m3_decode(a_code).astype(t)
    b = e4m3_decode(b_code).astype(t)
    c = np.matmul(a, b.T).astype(np.float32)
    s = np.float32(np.float32(scale_a) * np.float32(scale_b))
    return _cast_out((c * s).astype(np.float32), out_dtype)


# --------------------------------------------------------------------------------------
# error metric shared by every parity gate
# --------------------------------------------------------------------------------------

def max_rel_err(out: np.ndarray, ref: np.ndarray) -> float:
    """max |out - ref| / max |ref|: relative error normalised by the largest reference
    magnitude (elementwise relative error is unbounded at near-zero outputs)."""
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = float(np.max(np.abs(ref)))
    if den == 0.0:
        return float(np.max(np.abs(out)))
    return float(np.max(np.abs(out - ref)) / den)


# --------------------------------------------------------------------------------------
# seeded synthetic inputs: one recipe used on both machines
# --------------------------------------------------------------------------------------

def make_inputs(seed: int, m: int, k: int, n: int, w_std: float = 0.02):
    """A ~ N(0,1) [m,k] float32 drawn first, then W ~ N(0, w_std^2) [k,n] float32."""
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.standard_normal((k, n), dtype=np.float32)
    w *= np.float32(w_std)
    return a, w
