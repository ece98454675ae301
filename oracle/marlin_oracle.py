"""CPU oracle for the Marlin W4A16 path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain numpy, the algorithms the reference implements
for its Marlin-family W4A16 GEMM.  It is the checker that the HIP kernels are
compared against.  Nothing in the shipped package imports it: only tests,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do.

Every function names the reference source it follows (paths relative to the
reference checkout).  How each function is pinned (none is "parity unpinned"):

* ScalarType ids           closed-form bitfield + min/max table of
                           tests/test_scalartype.py:10-25
* gptq/awq/col packing     unpack(pack(x)) == x, brute force against a
                           per-element python loop
* Marlin weight layout     two independent derivations must agree: the
                           reshape/permute/perm-table recipe
                           (marlin_utils_test.py:31-121) and the per-thread
                           index arithmetic of the CUDA repack kernels
                           (gptq_marlin_repack.cu:129-209,
                           awq_marlin_repack.cu:89-157); bijection on nibbles
* scale/zp/bias permutes   closed-form index tables, permutation property,
                           inverse round trip
* dequantised values       exhaustive over all 16 codes x all finite fp16 /
                           bf16 scales of a sample, against exact rational
                           arithmetic (fractions) rounded to nearest even
* GEMM reference           textbook: dequantise then fp32 matmul; special
                           cases that reduce to row sums / column picks
* moe_align_block_size     the literal example in
                           fused_moe/moe_align_block_size.py:60-73 and set
                           equality per expert
                           (tests/kernels/moe/test_moe_align_block_size.py)
* gfx950 layout            this build's own format: inverse round trip and
                           decode-to-(K,N) equality with the Marlin decode
* 8-bit weights (W8A16)    the same pinning as the 4-bit functions: recipe
                           (get_weight_perm(8), interleave [0,2,1,3]) against
                           the repack kernel's arithmetic
                           (gptq_marlin_repack.cu:129-236), bijection on
                           bytes, round trips, exhaustive dequantisation over
                           256 codes
* fp8 weights (W8A16-fp8)  the table of the 254 finite codes against torch's
                           own float8_e4m3fn -> float32 conversion on the CPU
                           and hand values (0x38 = 1, 0x7e = 448, 0x01 =
                           2^-9); the kernel-side recipe (code read as a
                           16-bit float, scale with the exponent bias folded
                           in; dequant.h:320-380, marlin_utils_fp8.py:35-46)
                           against value * scale in exact rational arithmetic
                           rounded to nearest even, over all codes
* MXFP4 weights            the 16 values against the list in the OCP MX
                           format (0, 0.5, 1, 1.5, 2, 3, 4, 6 and negatives) and
                           against the reference's own test recipe (the code
                           moved into a float8_e4m3fn byte, converted by torch
                           on the CPU, times 2^6; marlin_utils_fp4.py:720-727);
                           scales 2^(e - 127) against torch's float8_e8m0fnu
                           conversion; the (0, 2, 1, 3) reorder is its own
                           inverse
* 8-bit activations        the 32 x 32 tile order (is_a_8bit) by the same two
                           derivations (get_weight_perm(4, True) recipe against
                           the repack kernel's arithmetic,
                           gptq_marlin_repack.cu:129-216), bijection, round
                           trips; the fp8 preprocess against the two formulas
                           the reference's tests state
                           (test_marlin_gemm.py:148-188) and its inverse; the
                           int8 GEMM against a per-element python loop with
                           the textbook dequantised matmul as the limit case
                           (all group scales equal); per_token_quant_int8
                           against hand values and the round trip bound
                           |x - q*s| <= s/2; MXFP4 with fp8 activations: the
                           byte a code becomes (dequant.h:474-490) decoded as
                           float8_e4m3fn equals 2^-6 times the code's value for
                           all 16 codes, which the scale bytes' + 6 undoes
* NVFP4 weights            the scale bytes (nvfp4_process_scales) decoded by both
                           of the kernel's readings (dequant.h:520-549: b << 7
                           as fp16, and sign / exponent / mantissa moved into a
                           bf16) against scale * 2^7 for every non-negative
                           float8_e4m3fn scale (torch's own conversion on the
                           CPU), the >= 2 cut, the scale factor against its
                           definition; global-scale processing against
                           2^(bias - 7); the dequantised weight times the
                           processed global scale against value * scale *
                           global scale in exact arithmetic
"""

from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------
# ScalarType ids  (aphrodite/scalar_type.py:129-156, csrc/core/scalar_type.hpp:131-164)
# --------------------------------------------------------------------------

NAN_REPR_IEEE_754 = 1  # scalar_type.py:65 default, also used for integer types


def scalar_type_id(exponent: int, mantissa: int, signed: bool, bias: int,
                   finite_values_only: bool = False,
                   nan_repr: int = NAN_REPR_IEEE_754) -> int:
    """Bitfield exponent[0:8] mantissa[8:16] signed[16] bias[17:49]
    finite_only[49] nan_repr[50:58] (scalar_type.py:137-150)."""
    val = 0
    off = 0
    for member, width in ((exponent, 8), (mantissa, 8), (int(signed), 1),
                          (bias, 32), (int(finite_values_only), 1),
                          (nan_repr, 8)):
        val |= (int(member) & ((1 << width) - 1)) << off
        off += width
    return val


UINT4B8_ID = scalar_type_id(0, 4, False, 8)      # scalar_types.uint4b8
UINT4_ID = scalar_type_id(0, 4, False, 0)        # scalar_types.uint4
UINT8B128_ID = scalar_type_id(0, 8, False, 128)  # scalar_types.uint8b128
NAN_REPR_EXTD_RANGE_MAX_MIN = 2                  # scalar_type.py:16
FLOAT8_E4M3FN_ID = scalar_type_id(4, 3, True, 0, True, NAN_REPR_EXTD_RANGE_MAX_MIN)  # scalar_type.py:314
FLOAT4_E2M1F_ID = scalar_type_id(2, 1, True, 0, True, 0)                              # scalar_type.py:327 (NanRepr.NONE)


def scalar_type_min_max(mantissa: int, signed: bool, bias: int):
    """Integer ScalarType.min()/max() (scalar_type.py:104-127,183-196):
    raw range minus bias."""
    size_bits = mantissa + int(signed)
    raw_max = (1 << mantissa) - 1
    raw_min = -(1 << (size_bits - 1)) if signed else 0
    return raw_min - bias, raw_max - bias


# --------------------------------------------------------------------------
# Checkpoint packings  (quant_utils.py:725-834)
# --------------------------------------------------------------------------

AWQ_ORDER = np.array([0, 2, 4, 6, 1, 3, 5, 7])  # quant_utils.py:823


def pack_rows(q: np.ndarray) -> np.ndarray:
    """GPTQ packing along K (quant_utils.py:725-746): word[k//8][n] holds
    q[k][n] at bits 4*(k%8)."""
    k, n = q.shape
    assert k % 8 == 0
    u = q.astype(np.uint32).reshape(k // 8, 8, n)
    out = np.zeros((k // 8, n), dtype=np.uint32)
    for i in range(8):
        out |= u[:, i, :] << np.uint32(4 * i)
    return out.view(np.int32)


def unpack_rows(packed: np.ndarray) -> np.ndarray:
    u = packed.view(np.uint32)
    kp, n = u.shape
    out = np.empty((kp, 8, n), dtype=np.int32)
    for i in range(8):
        out[:, i, :] = (u >> np.uint32(4 * i)) & np.uint32(0xF)
    return out.reshape(kp * 8, n)


def pack_cols(q: np.ndarray) -> np.ndarray:
    """Packing along N (quant_utils.py:749-772): word[k][n//8] holds q[k][n]
    at bits 4*(n%8)."""
    k, n = q.shape
    assert n % 8 == 0
    u = q.astype(np.uint32).reshape(k, n // 8, 8)
    out = np.zeros((k, n // 8), dtype=np.uint32)
    for i in range(8):
        out |= u[:, :, i] << np.uint32(4 * i)
    return out.view(np.int32)


def unpack_cols(packed: np.ndarray) -> np.ndarray:
    """quant_utils.py:775-803."""
    u = packed.view(np.uint32)
    k, npk = u.shape
    out = np.empty((k, npk, 8), dtype=np.int32)
    for i in range(8):
        out[:, :, i] = (u >> np.uint32(4 * i)) & np.uint32(0xF)
    return out.reshape(k, npk * 8)


gptq_pack = pack_rows  # quant_utils.py:806-812


def awq_pack(q: np.ndarray) -> np.ndarray:
    """AWQ packing (quant_utils.py:815-834): within every 8 columns, nibble
    position p holds column AWQ_ORDER[p]."""
    k, n = q.shape
    r = q.reshape(k, n // 8, 8)[:, :, AWQ_ORDER].reshape(k, n)
    return pack_cols(r)


def awq_unpack(packed: np.ndarray) -> np.ndarray:
    r = unpack_cols(packed)
    k, n = r.shape
    out = np.empty_like(r).reshape(k, n // 8, 8)
    out[:, :, AWQ_ORDER] = r.reshape(k, n // 8, 8)
    return out.reshape(k, n)


# --------------------------------------------------------------------------
# Marlin weight layout  (marlin_utils_test.py:31-121)
# --------------------------------------------------------------------------

def marlin_weight_perm_recipe() -> np.ndarray:
    """The 1024-entry gather table of a 16(k) x 64(n) tile for 4-bit weights
    and 16-bit activations, built the way get_weight_perm builds it
    (marlin_utils_test.py:89-121)."""
    table = []
    for lane in range(32):
        col = lane // 4
        one = []
        for block in (0, 1):
            for row in (2 * (lane % 4), 2 * (lane % 4) + 1,
                        2 * (lane % 4 + 4), 2 * (lane % 4 + 4) + 1):
                one.append(16 * row + col + 8 * block)
        for j in range(4):
            table.extend(p + 256 * j for p in one)
    perm = np.array(table)
    return perm.reshape(-1, 8)[:, AWQ_ORDER].ravel()


def marlin_pack_recipe(q: np.ndarray) -> np.ndarray:
    """(K,N) codes -> Marlin (K/16, 2N) int32 following marlin_permute_weights
    + marlin_weights (marlin_utils_test.py:31-66)."""
    k, n = q.shape
    assert k % 16 == 0 and n % 64 == 0
    perm = marlin_weight_perm_recipe()
    t = q.reshape(k // 16, 16, n // 16, 16).transpose(0, 2, 1, 3).reshape(k // 16, n * 16)
    t = t.reshape(-1, perm.size)[:, perm].reshape(t.shape)
    u = t.astype(np.uint32).reshape(k // 16, n * 2, 8)
    out = np.zeros((k // 16, n * 2), dtype=np.uint32)
    for i in range(8):
        out |= u[:, :, i] << np.uint32(4 * i)
    return out.view(np.int32)


def marlin_pack_closed_form(q: np.ndarray) -> np.ndarray:
    """Same layout derived from the repack kernels' per-thread arithmetic
    (gptq_marlin_repack.cu:129-209): tile (kt, nt) is 128 words at
    (kt*n_tiles+nt)*128; word lane*4+j, lane in [0,32), j = 16-column
    sub-tile; with c = lane//4, r0 = 2*(lane%4) the eight values
    vals[i] (i<4: column c, i>=4: column c+8; rows r0+{0,1,8,9}) are stored
    at nibble slots pack_idx = {0,2,4,6,1,3,5,7}."""
    k, n = q.shape
    assert k % 16 == 0 and n % 64 == 0
    kt_n, nt_n = k // 16, n // 64
    tile = q.reshape(kt_n, 16, nt_n, 4, 16).astype(np.uint32)  # [kt][r][nt][j][col]
    out = np.zeros((kt_n, nt_n, 32, 4), dtype=np.uint32)       # [kt][nt][lane][j]
    tc_offsets = (0, 1, 8, 9)
    pack_idx = (0, 2, 4, 6, 1, 3, 5, 7)
    for lane in range(32):
        c = lane // 4
        r0 = 2 * (lane % 4)
        vals = []
        for i in range(4):
            vals.append(tile[:, r0 + tc_offsets[i], :, :, c])
        for i in range(4):
            vals.append(tile[:, r0 + tc_offsets[i], :, :, c + 8])
        word = np.zeros_like(vals[0])
        for slot in range(8):
            word |= vals[pack_idx[slot]] << np.uint32(4 * slot)
        out[:, :, lane, :] = word
    return out.reshape(kt_n, nt_n * 128).view(np.int32)


marlin_pack = marlin_pack_closed_form


def marlin_unpack(packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    """Inverse of marlin_pack: Marlin (K/16, 2N) int32 -> (K,N) codes."""
    kt_n, nt_n = size_k // 16, size_n // 64
    u = packed.view(np.uint32).reshape(kt_n, nt_n, 32, 4)
    q = np.empty((kt_n, 16, nt_n, 4, 16), dtype=np.int32)
    tc_offsets = (0, 1, 8, 9)
    pack_idx = (0, 2, 4, 6, 1, 3, 5, 7)
    for lane in range(32):
        c = lane // 4
        r0 = 2 * (lane % 4)
        w = u[:, :, lane, :]
        for slot in range(8):
            i = pack_idx[slot]
            row = r0 + tc_offsets[i % 4]
            col = c + 8 * (i // 4)
            q[:, row, :, :, col] = (w >> np.uint32(4 * slot)) & np.uint32(0xF)
    return q.reshape(size_k, size_n)


def gptq_marlin_repack(b_q_weight: np.ndarray, perm: np.ndarray | None,
                       size_k: int, size_n: int) -> np.ndarray:
    """gptq_marlin_repack.cu:285-362: output row k takes source row perm[k]
    when perm is non-empty (:87-96,148-161)."""
    q = unpack_rows(b_q_weight)
    assert q.shape == (size_k, size_n)
    if perm is not None and perm.size > 0:
        q = q[perm.astype(np.int64), :]
    return marlin_pack(q)


def awq_marlin_repack(b_q_weight: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    """awq_marlin_repack.cu:228-290."""
    q = awq_unpack(b_q_weight)
    assert q.shape == (size_k, size_n)
    return marlin_pack(q)


# --------------------------------------------------------------------------
# 4-bit weights for 8-bit activations (is_a_8bit): 32(k) x 32(n) tiles
# --------------------------------------------------------------------------

A8_ORDER = np.array([0, 4, 1, 5, 2, 6, 3, 7])  # marlin_utils_test.py:108


def marlin_weight_perm_recipe_a8() -> np.ndarray:
    """The 1024-entry gather table of a 32(k) x 32(n) tile for 4-bit weights
    and 8-bit activations, built the way get_weight_perm(4, is_a_8bit=True)
    builds it (marlin_utils_test.py:71-88,106-120)."""
    table = []
    for lane in range(32):
        col = lane // 4
        one = []
        for block in (0, 1):
            for row in ([4 * (lane % 4) + t for t in range(4)]
                        + [4 * (lane % 4 + 4) + t for t in range(4)]):
                one.append(16 * row + col + 8 * block)
        for j in range(2):
            table.extend(p + 512 * j for p in one)
    perm = np.array(table)
    return perm.reshape(-1, 8)[:, A8_ORDER].ravel()


def marlin_pack_recipe_a8(q: np.ndarray) -> np.ndarray:
    """(K,N) codes -> Marlin (K/16, 2N) int32 for 8-bit activations following
    marlin_permute_weights(is_a_8bit=True) + marlin_weights
    (marlin_utils_test.py:31-66)."""
    k, n = q.shape
    assert k % 32 == 0 and n % 64 == 0
    perm = marlin_weight_perm_recipe_a8()
    t = q.reshape(k // 32, 32, n // 16, 16).transpose(0, 2, 1, 3).reshape(k // 16, n * 16)
    t = t.reshape(-1, perm.size)[:, perm].reshape(t.shape)
    u = t.astype(np.uint32).reshape(k // 16, n * 2, 8)
    out = np.zeros((k // 16, n * 2), dtype=np.uint32)
    for i in range(8):
        out |= u[:, :, i] << np.uint32(4 * i)
    return out.view(np.int32)


def _a8_word_sources(lane: int, warp: int):
    """Rows and column (inside a 32 x 32 tile) of the eight nibble slots of
    word lane*4 + warp, from the repack kernel's arithmetic
    (gptq_marlin_repack.cu:129-141,176-216 with is_a_8bit): column
    16*(warp/2) + 8*(warp%2) + lane/4; vals[i] = row 4*(lane%4) + i, vals[4+i]
    = that row + 16; slot s holds vals[{0,4,1,5,2,6,3,7}[s]]."""
    col = 16 * (warp // 2) + 8 * (warp % 2) + lane // 4
    rows = []
    for slot in range(8):
        i = (0, 4, 1, 5, 2, 6, 3, 7)[slot]
        rows.append(4 * (lane % 4) + (i % 4) + 16 * (i // 4))
    return rows, col


def marlin_pack_closed_form_a8(q: np.ndarray) -> np.ndarray:
    """Same layout from the repack kernels' per-thread arithmetic: tile
    (kt, nt) of 32 x 32 is 128 words at (kt*n_tiles + nt)*128, word
    lane*4 + warp."""
    k, n = q.shape
    assert k % 32 == 0 and n % 64 == 0
    kt_n, nt_n = k // 32, n // 32
    tile = q.reshape(kt_n, 32, nt_n, 32).astype(np.uint32)  # [kt][r][nt][c]
    out = np.zeros((kt_n, nt_n, 32, 4), dtype=np.uint32)
    for lane in range(32):
        for warp in range(4):
            rows, col = _a8_word_sources(lane, warp)
            word = np.zeros((kt_n, nt_n), dtype=np.uint32)
            for slot in range(8):
                word |= tile[:, rows[slot], :, col] << np.uint32(4 * slot)
            out[:, :, lane, warp] = word
    return out.reshape(k // 16, n * 2).view(np.int32)


marlin_pack_a8 = marlin_pack_closed_form_a8


def marlin_unpack_a8(packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    """Inverse of marlin_pack_a8."""
    kt_n, nt_n = size_k // 32, size_n // 32
    u = packed.view(np.uint32).reshape(kt_n, nt_n, 32, 4)
    q = np.empty((kt_n, 32, nt_n, 32), dtype=np.int32)
    for lane in range(32):
        for warp in range(4):
            rows, col = _a8_word_sources(lane, warp)
            for slot in range(8):
                q[:, rows[slot], :, col] = (u[:, :, lane, warp] >> np.uint32(4 * slot)) & np.uint32(0xF)
    return q.reshape(size_k, size_n)


def gptq_marlin_repack_a8(b_q_weight: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    """gptq_marlin_repack with is_a_8bit (no act-order: the kernel has
    static_assert(!is_a_8bit) under has_perm, gptq_marlin_repack.cu:147)."""
    q = unpack_rows(b_q_weight)
    assert q.shape == (size_k, size_n)
    return marlin_pack_a8(q)


def awq_marlin_repack_a8(b_q_weight: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    q = awq_unpack(b_q_weight)
    assert q.shape == (size_k, size_n)
    return marlin_pack_a8(q)


def marlin_pack8_recipe_a8(q: np.ndarray) -> np.ndarray:
    """8-bit codes in the order of 8-bit activations, by the recipe: the same gather table as
    for 4-bit codes before its interleave (get_weight_perm(8, True): interleave [0, 1, 2, 3],
    marlin_utils_test.py:111-115), four codes a word.  (K, N) -> (K/16, 4N) int32.  No GEMM of
    the reference takes this order (W8A8 is not a Marlin mode); the repack op produces it."""
    k, n = q.shape
    assert k % 32 == 0 and n % 64 == 0
    perm = marlin_weight_perm_recipe_a8().reshape(-1, 8)[:, np.argsort(A8_ORDER)].ravel()   # interleave undone
    t = q.reshape(k // 32, 32, n // 16, 16).transpose(0, 2, 1, 3).reshape(k // 16, n * 16)
    t = t.reshape(-1, perm.size)[:, perm].reshape(t.shape)
    u = t.astype(np.uint32).reshape(k // 16, n * 4, 4)
    out = np.zeros((k // 16, n * 4), dtype=np.uint32)
    for i in range(4):
        out |= u[:, :, i] << np.uint32(8 * i)
    return out.view(np.int32)


def marlin_pack8_closed_form_a8(q: np.ndarray) -> np.ndarray:
    """The same from the repack kernel's arithmetic (gptq_marlin_repack.cu:129-141,176-236 with
    is_a_8bit, num_bits 8): tile (kt, nt) of 32 x 32 is 256 words; word lane*8 + 2*warp + h holds
    column 8*warp + lane/4, rows 4*(lane%4) + {0,1,2,3} + 16h at bytes 0..3."""
    k, n = q.shape
    assert k % 32 == 0 and n % 64 == 0
    kt_n, nt_n = k // 32, n // 32
    tile = q.reshape(kt_n, 32, nt_n, 32).astype(np.uint32)
    out = np.zeros((kt_n, nt_n, 32, 4, 2), dtype=np.uint32)
    for lane in range(32):
        for warp in range(4):
            col = 8 * warp + lane // 4
            for h in range(2):
                word = np.zeros((kt_n, nt_n), dtype=np.uint32)
                for i in range(4):
                    word |= tile[:, 4 * (lane % 4) + i + 16 * h, :, col] << np.uint32(8 * i)
                out[:, :, lane, warp, h] = word
    return out.reshape(k // 16, n * 4).view(np.int32)


def gptq_marlin_repack8_a8(b_q_weight: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    q = unpack_rows8(b_q_weight)
    assert q.shape == (size_k, size_n)
    return marlin_pack8_closed_form_a8(q)


def marlin_a8_to_gfx950(marlin_packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    return gfx950_pack(marlin_unpack_a8(marlin_packed, size_k, size_n))


def int4_fp8_preprocess(q: np.ndarray, zeros: np.ndarray | None = None,
                        group_size: int | None = None) -> np.ndarray:
    """marlin_int4_fp8_preprocess.cu:13-66 on unpacked codes (the op works
    nibble by nibble, so the packing does not matter): sign and magnitude of
    code - z in a nibble; q >= z: q - z, else 15 - q.  z = 8 without zero
    points.  tests/kernels/quantization/test_marlin_gemm.py:148-188 states
    the same two formulas."""
    q = q.astype(np.int32)
    if zeros is None:
        return np.where(q >= 8, q - 8, 15 - q).astype(np.int32)
    z = np.repeat(zeros.astype(np.int32), group_size, axis=0)
    return np.where(q >= z, q - z, 15 - q).astype(np.int32)


def int4_fp8_preprocess_inverse(p: np.ndarray) -> np.ndarray:
    """Codes back from the preprocessed nibbles (no zero points)."""
    p = p.astype(np.int32)
    return np.where(p < 8, p + 8, 15 - p).astype(np.int32)


def marlin_permute_scales_a8(s: np.ndarray, size_k: int, size_n: int, group_size: int) -> np.ndarray:
    """marlin_utils.py:415-426 with is_a_8bit: always the single permutation."""
    return np.ascontiguousarray(s.reshape(-1, 32)[:, SCALE_PERM_SINGLE].reshape(-1, size_n))


def marlin_unpermute_scales_a8(s: np.ndarray, size_k: int, size_n: int, group_size: int) -> np.ndarray:
    out = np.empty_like(s).reshape(-1, 32)
    out[:, SCALE_PERM_SINGLE] = s.reshape(-1, 32)
    return np.ascontiguousarray(out.reshape(-1, size_n))


def marlin_zero_points_a8(zp: np.ndarray, num_groups: int, size_n: int) -> np.ndarray:
    """marlin_utils.py:456-477 with is_a_8bit: the scale permutation without
    the column interleave."""
    t = zp.reshape(-1, 64)[:, SCALE_PERM].reshape(num_groups, size_n)
    return pack_cols(t)


def marlin_unpack_zero_points_a8(zp_packed: np.ndarray, num_groups: int, size_n: int) -> np.ndarray:
    u = unpack_cols(zp_packed).reshape(-1, 64)
    out = np.empty_like(u)
    out[:, SCALE_PERM] = u
    return out.reshape(num_groups, size_n)


def awq_to_marlin_zero_points_a8(q_zp_packed: np.ndarray, num_groups: int, size_n: int) -> np.ndarray:
    return marlin_zero_points_a8(awq_unpack(q_zp_packed), num_groups, size_n)


def marlin_act_int8_process_scales(s32: np.ndarray):
    """marlin_utils.py:436-440: group scales as 16-bit integers
    round(s / max * 4096) and the factor max / 4096 that goes into the
    activation scales.  Returns (int16 array, float32 factor)."""
    top = np.float32(s32.max())
    factor = np.float32(np.float32(1.0 / 4096.0) * top)
    ints = np.rint((s32.astype(np.float32) / top) * np.float32(4096.0)).astype(np.int16)
    return ints, factor


def per_token_quant_int8(x32: np.ndarray):
    """int8_utils.py:70-93: scale = absmax / 127 per row (absmax at least
    1e-10), codes round-half-away(x * (127 / absmax)).  Returns (int8 (M,K),
    float32 (M,1))."""
    x = x32.astype(np.float32)
    absmax = np.maximum(np.max(np.abs(x), axis=1, keepdims=True), np.float32(1e-10)).astype(np.float32)
    scale = (absmax / np.float32(127.0)).astype(np.float32)
    y = x * (np.float32(127.0) / absmax).astype(np.float32)
    codes = (np.sign(y) * np.floor(np.abs(y) + np.float32(0.5))).astype(np.int8)
    return codes, scale


def gemm_w4a8_int8(a_q: np.ndarray, a_scales: np.ndarray, q: np.ndarray, group_size: int,
                   scales, dtype: str, zeros: np.ndarray | None = None,
                   bias32: np.ndarray | None = None) -> np.ndarray:
    """W4A8 with int8 activations (marlin_template.h:1302-1362,1869-1903,
    1955-1978).  Grouped (scales = the 16-bit integers of
    marlin_act_int8_process_scales, (groups, N)):
        c = sum_g scales[g][n] * sum_{k in g} a[m][k] * (q[k][n] - z)
    in 32-bit integer arithmetic (wrapping), out = float(c) * a_scales[m].
    Channelwise (group_size -1, scales = fp32 values of `dtype`, (1, N)):
        out = (float(sum_k a * (q - z)) * a_scales[m]) * scales[n].
    Then + bias in fp32 and one rounding to `dtype`.  z = 8 or the group's
    zero point.  Integer sums do not depend on the order, so a kernel matches
    this bit for bit."""
    m, k = a_q.shape
    n = q.shape[1]
    grouped = group_size not in (-1, k)
    gs = group_size if grouped else k
    groups = k // gs
    if zeros is None:
        centred = q.astype(np.int64) - 8
    else:
        centred = q.astype(np.int64) - np.repeat(zeros.astype(np.int64), gs, axis=0)
    a = a_q.astype(np.int64)
    total = np.zeros((m, n), dtype=np.int64)
    for g in range(groups):
        part = a[:, g * gs:(g + 1) * gs] @ centred[g * gs:(g + 1) * gs, :]
        part = ((part + 2**31) % 2**32) - 2**31
        if grouped:
            part = part * np.asarray(scales)[g].astype(np.uint16).astype(np.int64)[None, :]
        total = ((total + part + 2**31) % 2**32) - 2**31
    out = total.astype(np.int32).astype(np.float32) * a_scales.reshape(m, 1).astype(np.float32)
    if not grouped:
        out = out * np.asarray(scales, dtype=np.float32).reshape(1, n)
    if bias32 is not None:
        out = out + bias32.astype(np.float32)[None, :]
    return round_to_dtype(out.astype(np.float32), dtype)


def gemm_w4a8_fp8(a_fp8_32: np.ndarray, a_scales: np.ndarray, q: np.ndarray, group_size: int,
                  scales32: np.ndarray, zeros: np.ndarray | None = None,
                  bias32: np.ndarray | None = None) -> np.ndarray:
    """W4A8 with float8_e4m3fn activations (a_fp8_32: their values as fp32):
    out = (sum_g s[g][n] * sum_{k in g} a[m][k] * (q[k][n] - z)) * a_scales[m]
    (+ bias), in float64 here: a floating-point kernel is compared within a
    tolerance.  The reference keeps the weights as (q - z) * 2^-9 in fp8 and
    the scales times 512 (marlin_utils_test.py:156-158): the same product."""
    m, k = a_fp8_32.shape
    n = q.shape[1]
    grouped = group_size not in (-1, k)
    gs = group_size if grouped else k
    if zeros is None:
        centred = q.astype(np.float64) - 8.0
    else:
        centred = q.astype(np.float64) - np.repeat(zeros.astype(np.float64), gs, axis=0)
    w = centred * np.repeat(scales32.astype(np.float64), gs, axis=0)
    out = (a_fp8_32.astype(np.float64) @ w) * a_scales.reshape(m, 1).astype(np.float64)
    if bias32 is not None:
        out = out + bias32.astype(np.float64)[None, :]
    return out.astype(np.float32)


# --------------------------------------------------------------------------
# 8-bit weights (uint8b128, W8A16): same tile shape, four codes per word
# --------------------------------------------------------------------------

def pack_rows8(q: np.ndarray) -> np.ndarray:
    """GPTQ packing along K with 8-bit codes (quant_utils.py:725-746 with
    num_bits = 8): word[k//4][n] holds q[k][n] at bits 8*(k%4)."""
    k, n = q.shape
    assert k % 4 == 0
    u = q.astype(np.uint32).reshape(k // 4, 4, n)
    out = np.zeros((k // 4, n), dtype=np.uint32)
    for i in range(4):
        out |= u[:, i, :] << np.uint32(8 * i)
    return out.view(np.int32)


def unpack_rows8(packed: np.ndarray) -> np.ndarray:
    u = packed.view(np.uint32)
    kp, n = u.shape
    out = np.empty((kp, 4, n), dtype=np.int32)
    for i in range(4):
        out[:, i, :] = (u >> np.uint32(8 * i)) & np.uint32(0xFF)
    return out.reshape(kp * 4, n)


def marlin_weight_perm_recipe8() -> np.ndarray:
    """get_weight_perm(num_bits=8) (marlin_utils_test.py:69-121): the same
    1024-entry table as for 4 bits, interleaved in fours by [0, 2, 1, 3]."""
    table = []
    for lane in range(32):
        col = lane // 4
        one = []
        for block in (0, 1):
            for row in (2 * (lane % 4), 2 * (lane % 4) + 1,
                        2 * (lane % 4 + 4), 2 * (lane % 4 + 4) + 1):
                one.append(16 * row + col + 8 * block)
        for j in range(4):
            table.extend(p + 256 * j for p in one)
    return np.array(table).reshape(-1, 4)[:, [0, 2, 1, 3]].ravel()


def marlin_pack8_recipe(q: np.ndarray) -> np.ndarray:
    """(K,N) 8-bit codes -> Marlin (K/16, 4N) int32 following
    marlin_permute_weights + marlin_weights (marlin_utils_test.py:31-66)."""
    k, n = q.shape
    assert k % 16 == 0 and n % 64 == 0
    perm = marlin_weight_perm_recipe8()
    t = q.reshape(k // 16, 16, n // 16, 16).transpose(0, 2, 1, 3).reshape(k // 16, n * 16)
    t = t.reshape(-1, perm.size)[:, perm].reshape(t.shape)
    u = t.astype(np.uint32).reshape(k // 16, n * 4, 4)
    out = np.zeros((k // 16, n * 4), dtype=np.uint32)
    for i in range(4):
        out |= u[:, :, i] << np.uint32(8 * i)
    return out.view(np.int32)


def marlin_pack8_closed_form(q: np.ndarray) -> np.ndarray:
    """The repack kernel's arithmetic for num_bits = 8
    (gptq_marlin_repack.cu:129-236): tile (kt, nt) is 256 words; thread
    `lane` of warp j (16-column sub-tile) writes words lane*8 + 2j (column
    c = lane//4) and lane*8 + 2j + 1 (column c + 8); byte i of a word holds
    row 2*(lane%4) + {0, 1, 8, 9}[pack_idx[i]], pack_idx = {0, 2, 1, 3}."""
    k, n = q.shape
    assert k % 16 == 0 and n % 64 == 0
    kt_n, nt_n = k // 16, n // 64
    tile = q.reshape(kt_n, 16, nt_n, 4, 16).astype(np.uint32)  # [kt][r][nt][j][col]
    out = np.zeros((kt_n, nt_n, 32, 4, 2), dtype=np.uint32)    # [kt][nt][lane][j][half]
    tc_offsets = (0, 1, 8, 9)
    pack_idx = (0, 2, 1, 3)
    for lane in range(32):
        c = lane // 4
        r0 = 2 * (lane % 4)
        for half in (0, 1):
            word = np.zeros((kt_n, nt_n, 4), dtype=np.uint32)
            for i in range(4):
                word |= tile[:, r0 + tc_offsets[pack_idx[i]], :, :, c + 8 * half] << np.uint32(8 * i)
            out[:, :, lane, :, half] = word
    return out.reshape(kt_n, nt_n * 256).view(np.int32)


marlin_pack8 = marlin_pack8_closed_form


def marlin_unpack8(packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    kt_n, nt_n = size_k // 16, size_n // 64
    u = packed.view(np.uint32).reshape(kt_n, nt_n, 32, 4, 2)
    q = np.empty((kt_n, 16, nt_n, 4, 16), dtype=np.int32)
    tc_offsets = (0, 1, 8, 9)
    pack_idx = (0, 2, 1, 3)
    for lane in range(32):
        c = lane // 4
        r0 = 2 * (lane % 4)
        for half in (0, 1):
            w = u[:, :, lane, :, half]
            for i in range(4):
                q[:, r0 + tc_offsets[pack_idx[i]], :, :, c + 8 * half] = (w >> np.uint32(8 * i)) & np.uint32(0xFF)
    return q.reshape(size_k, size_n)


def gptq_marlin_repack8(b_q_weight: np.ndarray, perm: np.ndarray | None,
                        size_k: int, size_n: int) -> np.ndarray:
    """gptq_marlin_repack.cu:285-362 with num_bits = 8."""
    q = unpack_rows8(b_q_weight)
    assert q.shape == (size_k, size_n)
    if perm is not None and perm.size > 0:
        q = q[perm.astype(np.int64), :]
    return marlin_pack8(q)


# The gfx950 order for 8-bit codes: per strip a stream of 1-KiB blocks of 16
# rows each; block b = 2c + h belongs to 32-row chunk c.  Word j of lane L holds
# column 64*strip + 16*j + L%16 and rows 32c + 8*(L//16) + 4h + t, t = 0..3, row
# t at byte GFX950_BYTE[t], so that w & 0x00ff00ff is the row pair (0, 1) and
# (w >> 8) & 0x00ff00ff the pair (2, 3); blocks 2c and 2c+1 together give a
# lane the eight consecutive rows of one MFMA operand.

GFX950_BYTE = np.array([0, 2, 1, 3])


def gfx950_pack8(q: np.ndarray) -> np.ndarray:
    k, n = q.shape
    assert k % 32 == 0 and n % 64 == 0
    # [chunk][kb][h][t][strip][j][l]
    t = q.astype(np.uint32).reshape(k // 32, 4, 2, 4, n // 64, 4, 16)
    t = t.transpose(4, 0, 2, 1, 6, 5, 3)  # [strip][chunk][h][kb][l][j][t]
    out = np.zeros(t.shape[:-1], dtype=np.uint32)
    for row in range(4):
        out |= t[..., row] << np.uint32(8 * GFX950_BYTE[row])
    return out.reshape(-1).view(np.int32)


def gfx950_unpack8(packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    u = packed.view(np.uint32).reshape(size_n // 64, size_k // 32, 2, 4, 16, 4)
    t = np.empty(u.shape + (4,), dtype=np.int32)
    for row in range(4):
        t[..., row] = (u >> np.uint32(8 * GFX950_BYTE[row])) & np.uint32(0xFF)
    # [strip][chunk][h][kb][l][j][t] -> [chunk][kb][h][t][strip][j][l]
    return t.transpose(1, 3, 2, 6, 0, 5, 4).reshape(size_k, size_n)


def marlin8_to_gfx950(marlin_packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    return gfx950_pack8(marlin_unpack8(marlin_packed, size_k, size_n))


# --------------------------------------------------------------------------
# 8-bit floating-point weights: float8_e4m3fn codes in the 8-bit packings above
# (dequant.h:320-380; marlin_utils_fp8.py:35-46, 366-378, 591-631)
# --------------------------------------------------------------------------

def fp8_e4m3fn_values() -> np.ndarray:
    """The value of each of the 256 codes: sign bit, 4 exponent bits with bias
    7, 3 mantissa bits, subnormals at exponent 0, no infinities.  The codes
    0x7f and 0xff are NaN in the format; the kernels' bit trick reads them as
    the next step of the sequence, +-480, and so does this table."""
    code = np.arange(256)
    e, m = (code >> 3) & 15, code & 7
    mag = np.where(e == 0, m / 8.0 * 2.0 ** -6, (1 + m / 8.0) * 2.0 ** (e.astype(np.float64) - 7))
    return np.where(code & 0x80, -mag, mag).astype(np.float32)


FP8_EXPONENT_BIAS_SHIFT = {"fp16": 8, "bf16": 120}   # 2^(e-1) - 2^3 for e = 5 / 8 exponent bits


def fp8_fuse_exponent_bias(scales32: np.ndarray, dtype: str) -> np.ndarray:
    """marlin_utils_fp8.py:35-46: the scales the op receives, scales * 2^8
    (fp16) or * 2^120 (bf16), as values of `dtype` held in fp32."""
    return round_to_dtype((scales32.astype(np.float64) * 2.0 ** FP8_EXPONENT_BIAS_SHIFT[dtype]).astype(np.float32),
                          dtype)


def fp8_code_as_16bit_float(codes: np.ndarray, dtype: str) -> np.ndarray:
    """dequant.h:321-337, 357-374: the sign stays, the other seven bits move
    right by (exponent bits of `dtype`) - 4 below it; the 16-bit pattern read
    as `dtype` is value * 2^-8 (fp16) or value * 2^-120 (bf16).  Returned in
    fp32 (exact; bf16 subnormals are fp32 subnormals)."""
    c = codes.astype(np.uint32)
    shift = 1 if dtype == "fp16" else 4
    bits = ((c & 0x80) << 8) | (((c & 0x7F) << 8) >> shift)
    return from_bits16(bits.astype(np.uint16), dtype)


def dequantize_fp8(codes: np.ndarray, fused_scales32: np.ndarray, group_size: int, dtype: str) -> np.ndarray:
    """w[k][n] = round_to_dtype(code_as_16bit_float * fused_scale[g(k)][n]): the
    reference's one 16-bit multiply (marlin_template.h:1172-1299 with
    dequant_skip_flop, :353-357); the fp32 product of a 4-bit and an 11-bit
    significand is exact, so the rounding is the single one."""
    k, n = codes.shape
    rows = np.zeros(k, dtype=np.int64) if group_size in (-1, k) else np.arange(k) // group_size
    return round_to_dtype(fp8_code_as_16bit_float(codes, dtype) * fused_scales32.astype(np.float32)[rows, :], dtype)


# --------------------------------------------------------------------------
# MXFP4 weights: float4_e2m1f codes in the 4-bit packings above, one
# power-of-two scale per column and 32 rows, bf16 activations
# (dequant.h:397-470; marlin_utils_fp4.py:123-135, 217-290, 701-753)
# --------------------------------------------------------------------------

def fp4_e2m1_values() -> np.ndarray:
    """The value of each of the 16 codes: sign bit, 2 exponent bits with bias 1,
    1 mantissa bit, subnormal at exponent 0; no infinities, no NaN."""
    code = np.arange(16)
    e, m = (code >> 1) & 3, code & 1
    mag = np.where(e == 0, 0.5 * m, (1 + 0.5 * m) * 2.0 ** (e - 1))
    return np.where(code & 8, -mag, mag).astype(np.float32)


def mx_scale_values(exponent_bytes: np.ndarray) -> np.ndarray:
    """float8_e8m0fnu: 2^(e - 127) for e = 0..254 (255 is NaN, not used here)."""
    return np.ldexp(np.float32(1.0), exponent_bytes.astype(np.int32) - 127).astype(np.float32)


def mxfp4_process_scales(permuted: np.ndarray) -> np.ndarray:
    """marlin_utils_fp4.py:123-127: every four neighbours of the (already
    permuted) scale rows in the order 0, 2, 1, 3."""
    return permuted.reshape(-1, 4)[:, [0, 2, 1, 3]].reshape(permuted.shape)


def dequantize_mxfp4(codes: np.ndarray, exponent_bytes: np.ndarray, dtype: str = "bf16") -> np.ndarray:
    """w[k][n] = value(code[k][n]) * 2^(e[k // 32][n] - 127): a 2-bit significand
    times a power of two, exact in bf16."""
    k, n = codes.shape
    rows = np.arange(k) // 32
    return round_to_dtype(fp4_e2m1_values()[codes] * mx_scale_values(exponent_bytes)[rows, :], dtype)


def mxfp4_process_scales_a8(permuted_bytes: np.ndarray) -> np.ndarray:
    """marlin_utils_fp4.py:125-135 for float8_e4m3fn activations: no reorder
    inside the fours, every exponent byte plus 6 (the kernel holds a code as a
    float8_e4m3fn byte worth 2^-6 times the float4_e2m1f value: exponent bias
    7 against 1).  Bytes above 249 are refused, as the reference's assert does."""
    b = np.asarray(permuted_bytes).astype(np.int32)
    assert b.max() <= 249
    return (b + 6).astype(np.uint8)


def fp4_code_as_fp8_byte(code: np.ndarray) -> np.ndarray:
    """dequant.h:474-490: sign to bit 7, the two exponent bits and the mantissa
    bit to bits 4..2 of a float8_e4m3fn byte."""
    c = np.asarray(code).astype(np.uint8)
    return (((c & 8) << 4) | ((c & 7) << 2)).astype(np.uint8)


def fp8_e4m3fn_value(byte: np.ndarray) -> np.ndarray:
    """float8_e4m3fn: sign, 4 exponent bits (bias 7), 3 mantissa bits,
    subnormals at exponent 0 (NaN at 0x7f / 0xff not used here)."""
    b = np.asarray(byte).astype(np.int32)
    e, m = (b >> 3) & 15, b & 7
    mag = np.where(e == 0, m / 8.0 * 2.0 ** -6, (1 + m / 8.0) * 2.0 ** (e - 7.0))
    return np.where(b & 0x80, -mag, mag).astype(np.float32)


def gemm_w4a8_fp4(a_fp8_32: np.ndarray, a_scales: np.ndarray, codes: np.ndarray, exponent_bytes: np.ndarray,
                  bias32: np.ndarray | None = None) -> np.ndarray:
    """MXFP4 weights with float8_e4m3fn activations: out = (a @ w) * a_scales
    (+ bias) with w[k][n] = value(code) * 2^(e[k // 32][n] - 127), in float64
    (a floating-point kernel, compared within a tolerance).  `exponent_bytes`
    are the checkpoint's, before mxfp4_process_scales_a8."""
    m, k = a_fp8_32.shape
    w = fp4_e2m1_values()[codes].astype(np.float64) * np.repeat(
        mx_scale_values(exponent_bytes).astype(np.float64), 32, axis=0)
    out = (a_fp8_32.astype(np.float64) @ w) * a_scales.reshape(m, 1).astype(np.float64)
    if bias32 is not None:
        out = out + bias32.astype(np.float64)[None, :]
    return out.astype(np.float32)


# --------------------------------------------------------------------------
# NVFP4 weights: float4_e2m1f codes, one float8_e4m3fn scale per column and 16
# rows, one fp32 global scale, fp16 or bf16 activations
# (marlin_utils_fp4.py:37-151, 640-697; dequant.h:397-470, 518-549;
#  marlin_template.h:360-364, 1661-1665)
# --------------------------------------------------------------------------

NVFP4_EXPONENT_BIAS = {"fp16": 14, "bf16": 126}   # 2^(e-1) - 2^1 for e = 5 / 8 exponent bits (:143-149)


def nvfp4_scale_factor(scales32: np.ndarray, dtype: str) -> float:
    """marlin_utils_fp4.py:37-58: the power of two (>= 1) that lifts the largest
    scale times 2^7 towards 448 * 2^7; 1 for fp16 activations."""
    if dtype == "fp16":
        return 1.0
    ws = scales32.astype(np.float64) * 2.0 ** 7
    pos = ws[ws > 0]
    if pos.size and pos.max() < 448 * 2.0 ** 7:
        return float(2.0 ** np.floor(np.log2(448 * 2.0 ** 7 / pos.max())))
    return 1.0


def nvfp4_process_scales(permuted32: np.ndarray, dtype: str, scale_factor: float | None = None):
    """marlin_utils_fp4.py:61-120: (bytes, scale_factor).  The scales (values of
    float8_e4m3fn, >= 0, already in marlin_permute_scales order) go to fp16, every
    four neighbours into the order 0, 2, 1, 3, times the scale factor, times
    2^7; what is below 2 becomes 0; the byte is bits 14..7 of the fp16 number."""
    s = round_to_dtype(permuted32.astype(np.float32), "fp16")
    s = s.reshape(-1, 4)[:, [0, 2, 1, 3]].reshape(s.shape)
    if scale_factor is None:
        scale_factor = nvfp4_scale_factor(s, dtype)
    if scale_factor > 1.0:
        s = round_to_dtype((s.astype(np.float32) * np.float32(scale_factor)), "fp16")
    s = round_to_dtype(s * np.float32(2.0 ** 7), "fp16")
    s = np.where(s < 2, np.float32(0), s)
    bits = to_bits16(s, "fp16").astype(np.uint32)
    return ((bits << 1) >> 8 & 0xFF).astype(np.uint8), scale_factor


def nvfp4_scale_bytes_as_16bit_float(b: np.ndarray, dtype: str) -> np.ndarray:
    """dequant.h:520-549: what the kernel reads a scale byte as.  fp16: the bits
    b << 7.  bf16: bit 7 to bit 14, the other seven bits to bits 10..4.  Both are
    the fp16 reading's value when bit 7 is set (or the byte is 0)."""
    b = b.astype(np.uint32)
    if dtype == "fp16":
        return from_bits16((b << 7).astype(np.uint16), "fp16")
    return from_bits16((((b & 0x80) << 7) | ((b & 0x7F) << 4)).astype(np.uint16), "bf16")


def nvfp4_process_global_scale(global_scale: float, dtype: str, scale_factor: float = 1.0) -> np.float32:
    """marlin_utils_fp4.py:138-151 and :289-291: times 2^(exponent bias - 7), over
    the scale factor of the block scales; fp32."""
    return np.float32(np.float32(global_scale) * np.float32(2.0 ** (NVFP4_EXPONENT_BIAS[dtype] - 7))
                      / np.float32(scale_factor))


def nvfp4_kernel_scales(scale_bytes: np.ndarray, dtype: str) -> np.ndarray:
    """The block scales as this build's kernels take them: the kernel-side reading
    of a byte times 2^-(exponent bias), the factor the reference's dequantised
    code carries (dequant.h:397-470: a code read as fp16 / bf16 is value *
    2^-bias).  Plain marlin_permute_scales order (the 0, 2, 1, 3 reorder undone).
    Exact in `dtype` (held in fp32)."""
    v = nvfp4_scale_bytes_as_16bit_float(scale_bytes, dtype).astype(np.float64)
    v = v.reshape(-1, 4)[:, [0, 2, 1, 3]].reshape(v.shape)
    return (v * 2.0 ** -NVFP4_EXPONENT_BIAS[dtype]).astype(np.float32)


def dequantize_nvfp4(codes: np.ndarray, kernel_scales32: np.ndarray, dtype: str) -> np.ndarray:
    """w[k][n] = value(code[k][n]) * scale[k // 16][n] with the scales of
    nvfp4_kernel_scales in plain (K / 16, N) order: at most five significant
    bits, exact in fp16 and bf16 (the reference's one 16-bit multiply,
    marlin_template.h:1172-1299)."""
    k, n = codes.shape
    rows = np.arange(k) // 16
    return round_to_dtype(fp4_e2m1_values()[codes] * kernel_scales32.astype(np.float32)[rows, :], dtype)


# --------------------------------------------------------------------------
# Scale / zero-point / bias layouts  (marlin_utils.py:401-505)
# --------------------------------------------------------------------------

SCALE_PERM = np.array([i + 8 * j for i in range(8) for j in range(8)])           # :406-409
SCALE_PERM_SINGLE = np.array([2 * i + j for i in range(4)
                              for j in (0, 1, 8, 9, 16, 17, 24, 25)])          # :410-412


def marlin_permute_scales(s: np.ndarray, size_k: int, size_n: int, group_size: int) -> np.ndarray:
    """marlin_utils.py:415-426 (16-bit activations)."""
    if group_size < size_k and group_size != -1:
        out = s.reshape(-1, 64)[:, SCALE_PERM]
    else:
        out = s.reshape(-1, 32)[:, SCALE_PERM_SINGLE]
    return np.ascontiguousarray(out.reshape(-1, size_n))


def marlin_unpermute_scales(s: np.ndarray, size_k: int, size_n: int, group_size: int) -> np.ndarray:
    if group_size < size_k and group_size != -1:
        out = np.empty_like(s).reshape(-1, 64)
        out[:, SCALE_PERM] = s.reshape(-1, 64)
    else:
        out = np.empty_like(s).reshape(-1, 32)
        out[:, SCALE_PERM_SINGLE] = s.reshape(-1, 32)
    return np.ascontiguousarray(out.reshape(-1, size_n))


def marlin_permute_bias(b: np.ndarray) -> np.ndarray:
    """marlin_utils.py:429-433."""
    return np.ascontiguousarray(b.reshape(-1, 32)[:, SCALE_PERM_SINGLE].reshape(b.shape))


def marlin_unpermute_bias(b: np.ndarray) -> np.ndarray:
    out = np.empty_like(b).reshape(-1, 32)
    out[:, SCALE_PERM_SINGLE] = b.reshape(-1, 32)
    return np.ascontiguousarray(out.reshape(b.shape))


def marlin_zero_points(zp: np.ndarray, num_groups: int, size_n: int) -> np.ndarray:
    """marlin_utils.py:456-477: (groups, N) codes -> (groups, N/8) int32."""
    t = zp.reshape(-1, 64)[:, SCALE_PERM]
    t = t.reshape(-1, 8)[:, AWQ_ORDER].reshape(num_groups, size_n)
    return pack_cols(t)


def marlin_unpack_zero_points(zp_packed: np.ndarray, num_groups: int, size_n: int) -> np.ndarray:
    t = unpack_cols(zp_packed).reshape(-1, 8)
    u = np.empty_like(t)
    u[:, AWQ_ORDER] = t
    u = u.reshape(-1, 64)
    out = np.empty_like(u)
    out[:, SCALE_PERM] = u
    return out.reshape(num_groups, size_n)


def awq_to_marlin_zero_points(q_zp_packed: np.ndarray, num_groups: int, size_n: int) -> np.ndarray:
    """marlin_utils.py:480-505: AWQ-packed zero points -> Marlin layout."""
    return marlin_zero_points(awq_unpack(q_zp_packed), num_groups, size_n)


def stable_sort_g_idx(g_idx: np.ndarray):
    """marlin_sort_g_idx (marlin_utils.py:401-403) with a stable sort, so the
    tie order is fixed; the same perm must reach repack and GEMM."""
    order = np.argsort(g_idx, kind="stable").astype(np.int32)
    return g_idx[order], order


# --------------------------------------------------------------------------
# gfx950 streaming layout (this build's own format; no reference counterpart)
# --------------------------------------------------------------------------
# The (K,N) code matrix is cut into 64-column strips; a strip is a contiguous
# run of K/32 one-KiB chunks, chunk c covering rows [32c, 32c+32).  Inside a
# chunk, wavefront lane L (0..63) owns 16 bytes = words j=0..3.  Word j of lane
# L holds column 64*strip + 16*j + (L % 16) and the eight rows
# 32c + 8*(L // 16) + t, t = 0..7, with row t at nibble slot GFX950_SLOT[t], so
# that (w >> 4*i) & 0x000f000f yields the row pair (2i, 2i+1) in the low / high
# 16-bit halves: exactly one v_mfma_f32_16x16x32 operand register each.

GFX950_SLOT = np.array([0, 4, 1, 5, 2, 6, 3, 7])  # slot of row t; inverse of AWQ_ORDER


def gfx950_pack(q: np.ndarray) -> np.ndarray:
    k, n = q.shape
    assert k % 32 == 0 and n % 64 == 0
    # [strip][chunk][kb][t][j][l]
    t = q.astype(np.uint32).reshape(k // 32, 4, 8, n // 64, 4, 16)
    t = t.transpose(3, 0, 1, 5, 4, 2)  # [strip][chunk][kb][l][j][t]
    out = np.zeros(t.shape[:-1], dtype=np.uint32)
    for row in range(8):
        out |= t[..., row] << np.uint32(4 * GFX950_SLOT[row])
    return out.reshape(-1).view(np.int32)


def gfx950_unpack(packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    u = packed.view(np.uint32).reshape(size_n // 64, size_k // 32, 4, 16, 4)
    t = np.empty(u.shape + (8,), dtype=np.int32)
    for row in range(8):
        t[..., row] = (u >> np.uint32(4 * GFX950_SLOT[row])) & np.uint32(0xF)
    # [strip][chunk][kb][l][j][t] -> [chunk][kb][t][strip][j][l]
    return t.transpose(1, 2, 5, 0, 4, 3).reshape(size_k, size_n)


def marlin_to_gfx950(marlin_packed: np.ndarray, size_k: int, size_n: int) -> np.ndarray:
    return gfx950_pack(marlin_unpack(marlin_packed, size_k, size_n))


# --------------------------------------------------------------------------
# 16-bit float helpers
# --------------------------------------------------------------------------

def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16 (uint16 bit patterns)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (u + np.uint64(0x7FFF) + ((u >> np.uint64(16)) & np.uint64(1))) >> np.uint64(16)
    out = rounded.astype(np.uint16)
    nan = np.isnan(np.asarray(x, dtype=np.float32))
    if np.any(nan):
        out = np.where(nan, np.uint16(0x7FC0), out)
    return out


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_to_dtype(x32: np.ndarray, dtype: str) -> np.ndarray:
    """fp32 -> fp16/bf16 (RNE) -> fp32."""
    if dtype == "fp16":
        return np.asarray(x32, dtype=np.float32).astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_bits_to_f32(f32_to_bf16_bits(x32))
    raise ValueError(dtype)


def to_bits16(x32: np.ndarray, dtype: str) -> np.ndarray:
    """fp32 values (already representable) -> uint16 storage bits."""
    if dtype == "fp16":
        return np.asarray(x32, dtype=np.float32).astype(np.float16).view(np.uint16)
    return f32_to_bf16_bits(x32)


def from_bits16(b: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "fp16":
        return np.asarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)
    return bf16_bits_to_f32(b)


# --------------------------------------------------------------------------
# Dequantisation  (dequant.h:107-216, marlin_template.h:107-142,1182-1299;
#                  python twin quant_utils.py:646-648)
# --------------------------------------------------------------------------

def dequantize(q: np.ndarray, scales32: np.ndarray, group_size: int, dtype: str,
               zeros: np.ndarray | None = None, g_idx: np.ndarray | None = None,
               num_bits: int = 4) -> np.ndarray:
    """w[k][n] = round_to_dtype((q[k][n] - z) * s[g(k)][n]) with z = 8
    (uint4b8) or the group's zero point (uint4); s is a value of `dtype`
    held as fp32; one rounding, to nearest even.  (q - z) is a small integer,
    s has at most 11 significant bits, so the fp32 product is exact and the
    single rounding happens in round_to_dtype.  g(k) = k // group_size, or
    g_idx[k] when given (act-order)."""
    k, n = q.shape
    if g_idx is not None:
        rows = np.asarray(g_idx, dtype=np.int64)
    elif group_size in (-1, k):
        rows = np.zeros(k, dtype=np.int64)
    else:
        rows = np.arange(k) // group_size
    s = scales32.astype(np.float32)[rows, :]
    if zeros is None:
        centred = q.astype(np.int32) - (8 if num_bits == 4 else 128)   # uint4b8 / uint8b128
    else:
        centred = q.astype(np.int32) - zeros.astype(np.int32)[rows, :]
    return round_to_dtype(centred.astype(np.float32) * s, dtype)


def gemm_reference(a32: np.ndarray, w32: np.ndarray, bias32: np.ndarray | None = None) -> np.ndarray:
    """Dequantise-then-fp32-matmul reference (tests/kernels/quantization/
    test_marlin_gemm.py:483-491 uses torch.matmul(a, w_ref))."""
    out = a32.astype(np.float32) @ w32.astype(np.float32)
    if bias32 is not None:
        out = out + bias32.astype(np.float32)[None, :]
    return out


def gemm_tolerance_ok(out32: np.ndarray, ref32: np.ndarray):
    """The acceptance rule of this build: max|err| <= 1e-2*max|ref| and
    |err| <= 1e-2*max|ref| + 1e-2*|ref| elementwise.  Returns (ok, max_err,
    max_ref)."""
    err = np.abs(out32.astype(np.float64) - ref32.astype(np.float64))
    max_ref = float(np.max(np.abs(ref32))) if ref32.size else 0.0
    max_err = float(np.max(err)) if err.size else 0.0
    ok = max_err <= 1e-2 * max_ref + 1e-30
    ok = ok and bool(np.all(err <= 1e-2 * max_ref + 1e-2 * np.abs(ref32) + 1e-30))
    return ok, max_err, max_ref


# --------------------------------------------------------------------------
# Seeded synthetic layers (shapes and distributions of the benchmark configs)
# --------------------------------------------------------------------------

def make_layer(seed: int, size_k: int, size_n: int, group_size: int, dtype: str,
               zero_points: bool = False, act_order: bool = False):
    """Codes uniform over 0..15, scales uniform in [1e-3, 1e-2] rounded to
    `dtype`, optional zero points uniform 0..15, optional act-order: a random
    row permutation mapped to groups (quant_utils.py:558-585)."""
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(size_k, size_n), dtype=np.int32)
    groups = 1 if group_size in (-1, size_k) else size_k // group_size
    s = round_to_dtype(rng.uniform(1e-3, 1e-2, size=(groups, size_n)).astype(np.float32), dtype)
    out = {"q": q, "scales": s, "group_size": group_size, "groups": groups}
    if zero_points:
        out["zeros"] = rng.integers(0, 16, size=(groups, size_n), dtype=np.int32)
    if act_order:
        rand_perm = rng.permutation(size_k)
        g_idx = (rand_perm // group_size).astype(np.int32)  # group of each checkpoint row
        out["g_idx"] = g_idx
    return out


def make_activations(seed: int, size_m: int, size_k: int, dtype: str, std: float = 1.0) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return round_to_dtype((rng.standard_normal((size_m, size_k)) * std).astype(np.float32), dtype)


# --------------------------------------------------------------------------
# MoE routing  (fused_moe/moe_align_block_size.py:11-101; golden in
# tests/kernels/moe/test_moe_align_block_size.py:85-159)
# --------------------------------------------------------------------------

def moe_align_block_size(topk_ids: np.ndarray, block_size: int, num_experts: int):
    numel = topk_ids.size
    max_padded = numel + num_experts * (block_size - 1)
    if numel < num_experts:
        max_padded = min(numel * block_size, max_padded)
    flat = topk_ids.reshape(-1).astype(np.int64)
    sorted_ids = np.full(max_padded, numel, dtype=np.int32)
    expert_ids = np.full((max_padded + block_size - 1) // block_size, -1, dtype=np.int32)
    pos = 0
    blk = 0
    for e in range(num_experts):
        toks = np.nonzero(flat == e)[0].astype(np.int32)  # ascending = stable
        if toks.size == 0:
            continue
        nblk = (toks.size + block_size - 1) // block_size
        sorted_ids[pos:pos + toks.size] = toks
        expert_ids[blk:blk + nblk] = e
        pos += nblk * block_size
        blk += nblk
    return sorted_ids, expert_ids, np.array([pos], dtype=np.int32)


def batched_moe_align_block_size(max_tokens_per_batch: int, block_size: int, expert_num_tokens):
    """Tokens already batched by expert (csrc/libtorch_stable/moe/
    moe_align_sum_kernels.cu:26-82): batch b owns ceil(n_b / bs) blocks laid end
    to end; slot i of its range holds row b * max_tokens + i for i < n_b, the
    rest B * max_tokens; blocks of no batch hold expert -1."""
    n = [int(x) for x in expert_num_tokens]
    batches = len(n)
    per_batch = -(-max_tokens_per_batch // block_size) * block_size
    sentinel = batches * max_tokens_per_batch
    sorted_ids = np.full(batches * per_batch, sentinel, dtype=np.int32)
    expert_ids = np.full(batches * per_batch // block_size, -1, dtype=np.int32)
    at = 0
    for b, count in enumerate(n):
        padded = -(-count // block_size) * block_size
        sorted_ids[at:at + count] = b * max_tokens_per_batch + np.arange(count)
        expert_ids[at // block_size:(at + padded) // block_size] = b
        at += padded
    return sorted_ids, expert_ids, np.array([at], dtype=np.int32)


def moe_block_size_rule(m: int, topk: int, num_experts: int) -> int:
    """fused_marlin_moe block size choice (experts/marlin_moe.py:322-329)."""
    for bs in (8, 16, 32, 48, 64):
        if m * topk / num_experts / bs < 0.9:
            return bs
    return 64


def moe_activation(name: str, x32: np.ndarray, dtype: str, clamp_limit: float | None = None, alpha: float = 1.0,
                   beta: float = 0.0, situ_beta: float | None = None, situ_linear_beta: float | None = None) -> np.ndarray:
    """The activation between the two grouped GEMMs of the fused mixture-of-experts layer
    (apply_moe_activation, aphrodite/model_executor/layers/fused_moe/activation.py:128-205):
    x32 holds values of `dtype`, [rows, 2 d] for a gated activation (gate half then up half;
    "swigluoai": gate and up alternate), [rows, d] for one without a gate; returns [rows, d]
    values of `dtype`.  Every rounding to `dtype` the reference's kernels make is made here,
    exp / tanh / erf in float64 (a kernel's float32 functions may differ in the last place):
      silu                  T(T(g / (1 + e^-g)) * u)      csrc/libtorch_stable/activation_kernels.cu:28-76,157-160
      silu + clamp_limit,   g = T(min(gate, limit)), u = clamp(up, +-limit):
      swigluoai_uninterleave  T(T(g / (1 + e^(-alpha g))) * (u + beta))      (:60-75; silu_and_mul_with_clamp)
      gelu, gelu_tanh       T(T(gelu(g)) * u)             (:172-215)
      swigluoai             g = min(gate, 7), u = clamp(up, +-7): T((u + 1) g / (1 + e^(-1.702 g)))   (:412-423)
      situ                  T(b tanh(g / b) / (1 + e^-g) * (lb > 0 ? lb tanh(u / lb) : u))   (:489-510)
      swiglustep            T(min(g sigmoid(g), 7) * clamp(u, +-7))    (layers/activation.py:27-52)
      silu_no_mul, gelu_no_mul, gelu_tanh_no_mul   T(f(x));   relu2_no_mul   T(T(max(x, 0))^2)"""
    x = np.asarray(x32, dtype=np.float64)

    def rnd(v):
        return round_to_dtype(np.asarray(v, dtype=np.float64).astype(np.float32), dtype).astype(np.float64)

    def erf(v):
        from math import erf as erf1
        return np.vectorize(erf1)(v)

    # the two GELU forms in float32 step by step, as the kernels write them: far in the negative
    # tail 1 + erf(..) cancels, and what is left depends on the float32 sum, not on the function
    def gelu(v):
        f = v.astype(np.float32)
        e = erf((f * np.float32(0.70710678118654752440)).astype(np.float64)).astype(np.float32)
        return (f * np.float32(0.5) * (np.float32(1.0) + e)).astype(np.float64)

    def gelu_tanh(v):
        f = v.astype(np.float32)
        inner = np.float32(0.79788456080286535588) * (f + np.float32(0.044715) * (f * f * f))
        t = np.tanh(inner.astype(np.float64)).astype(np.float32)
        return (np.float32(0.5) * f * (np.float32(1.0) + t)).astype(np.float64)

    if name.endswith("_no_mul"):
        if name == "silu_no_mul":
            return rnd(x / (1.0 + np.exp(-x))).astype(np.float32)
        if name == "gelu_no_mul":
            return rnd(gelu(x)).astype(np.float32)
        if name == "gelu_tanh_no_mul":
            return rnd(gelu_tanh(x)).astype(np.float32)
        if name == "relu2_no_mul":
            return rnd(rnd(np.maximum(x, 0.0)) ** 2).astype(np.float32)
        raise ValueError(name)
    d = x.shape[-1] // 2
    if name == "swigluoai":
        g, u = x[..., 0::2], x[..., 1::2]
        g = np.minimum(g, 7.0)
        u = np.clip(u, -7.0, 7.0)
        return rnd((u + 1.0) * g / (1.0 + np.exp(-g * np.float64(np.float32(1.702))))).astype(np.float32)
    g, u = x[..., :d], x[..., d:]
    if name == "silu" and clamp_limit is None:
        return rnd(rnd(g / (1.0 + np.exp(-g))) * u).astype(np.float32)
    if name in ("silu", "swigluoai_uninterleave"):
        if clamp_limit is None:
            raise ValueError("swigluoai_uninterleave needs clamp_limit")
        a, b = (1.0, 0.0) if name == "silu" else (np.float64(np.float32(alpha)), np.float64(np.float32(beta)))
        lim = np.float64(np.float32(clamp_limit))
        gc = rnd(np.minimum(g, lim))
        uc = np.clip(u, -lim, lim)
        act = rnd(gc / (1.0 + np.exp(-gc * a)))
        return rnd(act * (uc + b)).astype(np.float32)
    if name == "gelu":
        return rnd(rnd(gelu(g)) * u).astype(np.float32)
    if name == "gelu_tanh":
        return rnd(rnd(gelu_tanh(g)) * u).astype(np.float32)
    if name == "situ":
        b = np.float64(np.float32(situ_beta))
        gate_out = b * np.tanh(g / b) / (1.0 + np.exp(-g))
        up_out = u
        if situ_linear_beta is not None and situ_linear_beta > 0:
            lb = np.float64(np.float32(situ_linear_beta))
            up_out = lb * np.tanh(u / lb)
        return rnd(gate_out * up_out).astype(np.float32)
    if name == "swiglustep":
        return rnd(np.minimum(g / (1.0 + np.exp(-g)), 7.0) * np.clip(u, -7.0, 7.0)).astype(np.float32)
    raise ValueError(name)


def moe_gemm_reference(a32: np.ndarray, w32_per_expert, sorted_ids: np.ndarray,
                       expert_ids: np.ndarray, num_post_pad: int, block_size: int,
                       top_k: int, size_m: int, topk_weights: np.ndarray | None,
                       dtype: str) -> np.ndarray:
    """moe_wna16_marlin_gemm semantics (moe/marlin_moe_wna16/ops.cu:544-897,
    marlin_template.h(moe):471-570,1883-1909): for every valid slot id of
    block b, C[id] = A[id // top_k] @ W[expert_ids[b]], rounded to dtype, then
    optionally multiplied by dtype(topk_weights[id]) in dtype arithmetic."""
    n = w32_per_expert[0].shape[1]
    out = np.zeros((size_m * top_k, n), dtype=np.float32)
    for b in range(num_post_pad // block_size):
        e = int(expert_ids[b])
        if e < 0:
            continue
        ids = sorted_ids[b * block_size:(b + 1) * block_size]
        ids = ids[ids < size_m * top_k]
        if ids.size == 0:
            continue
        rows = a32[ids // top_k, :]
        c = round_to_dtype(rows @ w32_per_expert[e], dtype)
        if topk_weights is not None:
            wts = round_to_dtype(topk_weights.reshape(-1)[ids].astype(np.float32), dtype)
            c = round_to_dtype(c * wts[:, None], dtype)
        out[ids, :] = c
    return out


def moe_gemm_w4a8_int8(a_q: np.ndarray, a_scales: np.ndarray, experts, sorted_ids: np.ndarray,
                       expert_ids: np.ndarray, num_post_pad: int, block_size: int, top_k: int,
                       topk_weights: np.ndarray | None, dtype: str) -> np.ndarray:
    """moe_wna16_marlin_gemm with int8 activations: for every valid slot id of block b,
    C[id] = gemm_w4a8_int8(row id // top_k of A with its scale, expert expert_ids[b]),
    then optionally times dtype(topk_weights[id]) in dtype arithmetic
    (moe/marlin_moe_wna16/marlin_template.h:471-560,622-650,1883-1909).  `experts`: one
    dict per expert with q, group_size, scales, zeros (or None), bias32 (or None)."""
    size_m = a_q.shape[0]
    n = experts[0]["q"].shape[1]
    out = np.zeros((size_m * top_k, n), dtype=np.float32)
    for b in range(num_post_pad // block_size):
        e = int(expert_ids[b])
        if e < 0 or e >= len(experts):
            continue
        ids = sorted_ids[b * block_size:(b + 1) * block_size]
        ids = ids[ids < size_m * top_k]
        if ids.size == 0:
            continue
        rows = ids // top_k
        ex = experts[e]
        c = gemm_w4a8_int8(a_q[rows], a_scales.reshape(-1)[rows], ex["q"], ex["group_size"], ex["scales"], dtype,
                           ex.get("zeros"), ex.get("bias32"))
        if topk_weights is not None:
            wts = round_to_dtype(topk_weights.reshape(-1)[ids].astype(np.float32), dtype)
            c = round_to_dtype(c * wts[:, None], dtype)
        out[ids, :] = c
    return out


# --------------------------------------------------------------------------
# CPU baseline of the layer: int4 dequantise + torch.matmul in fp32
# --------------------------------------------------------------------------

def cpu_layer_baseline(q_packed_rows: np.ndarray, scales32: np.ndarray, a32: np.ndarray,
                       group_size: int, threads: int, repeats: int = 5, warmup: int = 2):
    """Times W = (unpack(q) - 8) * s (fp32) followed by torch.matmul(A, W) in
    fp32 on `threads` host threads.  Returns (seconds_dequant_plus_matmul,
    seconds_matmul_only, output)."""
    import time

    import torch

    torch.set_num_threads(threads)
    qp = torch.from_numpy(q_packed_rows.view(np.int32).copy())
    s = torch.from_numpy(scales32.astype(np.float32))
    a = torch.from_numpy(a32.astype(np.float32))
    shifts = torch.arange(0, 32, 4, dtype=torch.int32).view(1, 8, 1)

    def dequant():
        nib = (qp.unsqueeze(1) >> shifts) & 0xF            # (K/8, 8, N)
        w = (nib.reshape(-1, qp.shape[1]).float() - 8.0)
        return w * s.repeat_interleave(group_size, dim=0)

    w = dequant()
    for _ in range(warmup):
        out = a @ dequant()
    t_full = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        out = a @ dequant()
        t_full.append(time.perf_counter() - t0)
    t_mm = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        out2 = a @ w
        t_mm.append(time.perf_counter() - t0)
    del out2
    return float(np.median(t_full)), float(np.median(t_mm)), out.numpy()
