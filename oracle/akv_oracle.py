"""CPU restatement (NumPy) of AlignedKV's split-precision K/V cache and decode attention.

THIS IS TEST INFRASTRUCTURE, NOT THE PRODUCT.  Only tests, the smoke check and the benchmark's
CPU-baseline leg may import it; the product path (alignedkv_amd) never does.

Every function restates one piece of the reference and cites the file:line it follows
(paths relative to the reference checkout).  Accumulation is fp32 (the reference kernels
accumulate in fp16 with sequential __hfma2; exact fp16 bits of those sums are "parity unpinned",
nothing in the reference pins them).  Integer / byte work (plane split, nibble packing, level
decisions, exponent bookkeeping) is restated bit for bit, including the reference's quirks.

What pins each function (tests/test_oracle_*.py):
  split_fp16 / reconstruct      exhaustive over all 65536 fp16 patterns, level-0 round trip
  k_cache_save / v_cache_save   brute-force flat-index loops written from the kernel's index
                                expressions on tiny shapes + the independent C restatement
  k_levels / v_levels           exhaustive tables against scalar C-style integer arithmetic
  k_cache_compute / v_cache_*   level-0 (reference=True) == dense float64 matmul on the
                                original fp16 values; substituted levels == matmul on values
                                truncated by closed form; cross-check with the C restatement
  bucket_max / amin / colmax    brute force on tiny inputs, closed forms
  k_sum_and_max                 nested scalar loops on a tiny shape, known answers (tests/test_oracle_helpers.py)
  softmax_fp32_to_half          torch.softmax(x.float()).half() on rows with -inf tails (<= 1 fp16 ulp, >= 99.9 % bit
                                equal), float64 closed form, known answers
  dense_attention               torch's fp16 matmul / fp32 softmax restatement of model/Llama_AlignedKV.py:130-139,
                                float64 attention, a one-hot known answer
fp16 tensors are carried as np.uint16 bit patterns unless stated otherwise.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np

COLUMN_BLOCK = 64  # extension/k_cache_file.py:5-6  (bits_in_a_channel // 4)
TOP_MAX_K = 32     # extension/v_cache_file.py:16
FP16_EXP_BIAS = 15  # extension/v_cache_file.py:156


def cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


# --------------------------------------------------------------------------------------
# bit-level pieces
# --------------------------------------------------------------------------------------
def as_bits(x) -> np.ndarray:
    """fp16 array -> uint16 bit pattern (no copy when possible)."""
    x = np.asarray(x)
    if x.dtype == np.float16:
        return x.view(np.uint16)
    if x.dtype == np.uint16:
        return x
    raise TypeError(f"expected float16/uint16, got {x.dtype}")


def as_half(bits) -> np.ndarray:
    return np.asarray(bits, dtype=np.uint16).view(np.float16)


def split_fp16(bits):
    """fp16 bits -> (first_8, mid_4, last_4) fields.

    first_8 = byte 1 of the little-endian half (sign, 5 exponent bits, top 2 mantissa bits),
    mid_4 = mantissa bits 7:4, last_4 = mantissa bits 3:0.
    extension/csrc/K_cache.cu:49-56, extension/csrc/V_cache.cu:30-39.
    """
    bits = as_bits(bits)
    hi = (bits >> 8).astype(np.uint8)
    lo = (bits & 0xFF).astype(np.uint8)
    return hi, (lo >> 4).astype(np.uint8), (lo & 0x0F).astype(np.uint8)


def exponent_bits(bits) -> np.ndarray:
    """(x.view(int16) >> 10).to(uint8) & 0x1F -- extension/k_cache_file.py:77-78,98-99,136."""
    bits = as_bits(bits)
    return ((bits.view(np.int16) >> 10).astype(np.uint8) & np.uint8(0x1F)).astype(np.uint8)


def reconstruct(hi, mid, last, level):
    """fp16 bits the compute kernels feed into the FMA at a given fetch level.

    level 0: hi<<8 | mid<<4 | last      (all three planes)
    level 1: hi<<8 | mid<<4 | 0x8       (last_4 replaced by the byte 0x88 of `trick`)
    level 2: hi<<8 | 0x80               (mid byte := 0x88, last byte := 0x00)
    extension/csrc/K_cache.cu:201-205,249-252, extension/csrc/V_cache.cu:198-202,250-253.
    """
    hi = np.asarray(hi, dtype=np.uint16)
    mid = np.asarray(mid, dtype=np.uint16)
    last = np.asarray(last, dtype=np.uint16)
    level = np.asarray(level)
    lo0 = (mid << 4) | last
    lo1 = (mid << 4) | np.uint16(0x8)
    lo2 = np.uint16(0x80)
    lo = np.where(level == 0, lo0, np.where(level == 1, lo1, lo2)).astype(np.uint16)
    return ((hi << 8) | lo).astype(np.uint16)


# --------------------------------------------------------------------------------------
# plane storage
# --------------------------------------------------------------------------------------
def k_planes_alloc(bsz, n_heads, max_seq_len, head_dim, d_block=COLUMN_BLOCK):
    """extension/k_cache_file.py:45-53."""
    nb = cdiv(max_seq_len, d_block)
    return (np.zeros((bsz, n_heads, nb, head_dim, d_block), np.uint8),
            np.zeros((bsz, n_heads, nb, head_dim, d_block // 2), np.uint8),
            np.zeros((bsz, n_heads, nb, head_dim, d_block // 2), np.uint8))


def v_planes_alloc(bsz, n_heads, max_seq_len, head_dim):
    """extension/v_cache_file.py:46-54."""
    return (np.zeros((bsz, n_heads, max_seq_len, head_dim), np.uint8),
            np.zeros((bsz, n_heads, max_seq_len, head_dim // 2), np.uint8),
            np.zeros((bsz, n_heads, max_seq_len, head_dim // 2), np.uint8))


def k_cache_save(first_8, mid_4, last_4, k_new_bits, n_blocks, d_block, start_pos, seqlen, tile_append=False):
    """In-place plane write of K.  k_new_bits: uint16 [B, seqlen, H, D].

    Prefill branch (start_pos == 0 or seqlen % d_block == 0): blocks z < n_blocks, tokens
    z*d_block .. min(z*d_block + d_block, seqlen); slot j of channel d goes to
    first_8[b,h,blk,d,j]; even j -> high nibble of byte j>>1, odd j -> low nibble; the nibble
    planes are updated with `+=` (uint8 wrap).  Decoding branch (seqlen == 1): one token at
    block start_pos // d_block, slot start_pos % d_block.
    extension/csrc/K_cache.cu:37-57 (prefill kernel), :83-93 (decoding kernel), :120-162 (dispatch).
    """
    k_new_bits = as_bits(k_new_bits)
    B, S, H, D = k_new_bits.shape
    assert S == seqlen
    hi, mid, last = split_fp16(k_new_bits)
    if start_pos == 0 or seqlen % d_block == 0:
        base_blk = start_pos // d_block
        for z in range(n_blocks):
            t0 = z * d_block
            t1 = min(t0 + d_block, seqlen)
            for seq in range(t0, t1):
                j = seq - t0
                first_8[:, :, z + base_blk, :, j] = hi[:, seq]
                mid_4[:, :, z + base_blk, :, j >> 1] += (mid[:, seq] << 4) >> ((j & 1) << 2)
                last_4[:, :, z + base_blk, :, j >> 1] += last[:, seq] << (4 - ((j & 1) << 2))
    elif seqlen == 1:
        blk = start_pos // d_block
        j = start_pos - blk * d_block
        first_8[:, :, blk, :, j] = hi[:, 0]
        mid_4[:, :, blk, :, j >> 1] += (mid[:, 0] << 4) >> ((j & 1) << 2)
        last_4[:, :, blk, :, j >> 1] += last[:, 0] << (4 - ((j & 1) << 2))
    elif tile_append and d_block % 64 == 0 and start_pos % 64 == 0 and seqlen % 64 == 0:
        # Not in the reference (it launches nothing here): whole 64-token tiles appended inside a larger block,
        # defined as seqlen applications of the single-token branch above.
        for i in range(seqlen):
            k_cache_save(first_8, mid_4, last_4, k_new_bits[:, i:i + 1], 1, d_block, start_pos + i, 1)


def v_cache_save(first_8, mid_4, last_4, v_new_bits, start_pos, seq_len):
    """In-place plane write of V.  v_new_bits: uint16 [B, S, H, D]; the first seq_len tokens are
    stored at rows start_pos .. start_pos+seq_len; channel 2c -> high nibble of byte c.
    extension/csrc/V_cache.cu:29-40,54-55.
    """
    if seq_len == 0:
        return
    v_new_bits = as_bits(v_new_bits)
    hi, mid, last = split_fp16(v_new_bits[:, :seq_len])
    hi = hi.transpose(0, 2, 1, 3)      # [B,H,S,D]
    mid = mid.transpose(0, 2, 1, 3)
    last = last.transpose(0, 2, 1, 3)
    sl = slice(start_pos, start_pos + seq_len)
    first_8[:, :, sl, :] = hi
    mid_4[:, :, sl, :] = (mid[..., 0::2] << 4) + mid[..., 1::2]
    last_4[:, :, sl, :] = (last[..., 0::2] << 4) + last[..., 1::2]


def k_planes_fields(first_8, mid_4, last_4, n_blocks):
    """Planes -> per-element (hi, mid, last) arrays shaped [B,H,n_blocks,D,d_block]."""
    hi = first_8[:, :, :n_blocks]
    m = mid_4[:, :, :n_blocks]
    l = last_4[:, :, :n_blocks]
    mid = np.empty(hi.shape, np.uint8)
    last = np.empty(hi.shape, np.uint8)
    mid[..., 0::2] = m >> 4
    mid[..., 1::2] = m & 0x0F
    last[..., 0::2] = l >> 4
    last[..., 1::2] = l & 0x0F
    return hi, mid, last


def v_planes_fields(first_8, mid_4, last_4, n_tokens):
    """Planes -> per-element (hi, mid, last) arrays shaped [B,H,n_tokens,D]."""
    hi = first_8[:, :, :n_tokens]
    m = mid_4[:, :, :n_tokens]
    l = last_4[:, :, :n_tokens]
    mid = np.empty(hi.shape, np.uint8)
    last = np.empty(hi.shape, np.uint8)
    mid[..., 0::2] = m >> 4
    mid[..., 1::2] = m & 0x0F
    last[..., 0::2] = l >> 4
    last[..., 1::2] = l & 0x0F
    return hi, mid, last


# --------------------------------------------------------------------------------------
# fetch-level decisions (the "masks")
# --------------------------------------------------------------------------------------
def k_levels(sum_u8, max_u8):
    """K fetch level per (b,h,channel).  sum_u8: uint8 [B,1,H,D] (or [B,H,D]),
    max_u8: uint8 [B,1,H,1] (or [B,H]).  diff = max - sum in uint8; >=8 -> 2, >=4 -> 1, else 0.
    extension/csrc/K_cache.cu:195,211,249-250.
    """
    s = np.asarray(sum_u8, np.uint8)
    B = s.shape[0]
    D = s.shape[-1]
    s = s.reshape(B, -1, D)
    m = np.asarray(max_u8, np.uint8).reshape(B, -1, 1)
    diff = (m - s).astype(np.uint8)   # uint8 wrap, as `unsigned char diff`
    return np.where(diff >= 8, 2, np.where(diff >= 4, 1, 0)).astype(np.uint8)


def v_levels(amin_u8, s_bits):
    """V fetch level per (b,h,token).  amin_u8: uint8 [B,H]; s_bits: uint16 [B,H,R].
    A = short(amin) << 10 (kept in a short), diff = short(A - short(bits(s)));
    diff >= 0x0800 -> 2, >= 0x0400 -> 1, else 0.
    extension/csrc/V_cache.cu:195-197,211,250-251.
    """
    a = np.asarray(amin_u8, np.uint8).astype(np.int32)
    A = ((a << 10) & 0xFFFF).astype(np.uint16).view(np.int16).astype(np.int32)
    sb = as_bits(s_bits).view(np.int16).astype(np.int32)
    diff = ((A[..., None] - sb) & 0xFFFF).astype(np.uint16).view(np.int16)
    return np.where(diff >= 0x0800, 2, np.where(diff >= 0x0400, 1, 0)).astype(np.uint8)


# --------------------------------------------------------------------------------------
# the three compute ops (fp32 accumulate)
# --------------------------------------------------------------------------------------
def half_scale(sqrt_dim: float) -> np.float32:
    """The kernel multiplies by __float2half2_rn(sqrt_dim): the scale is rounded to fp16 first.
    extension/csrc/K_cache.cu:306."""
    return np.float32(np.float16(np.float32(sqrt_dim)))


def k_cache_compute(first_8, mid_4, last_4, sum_u8, max_u8, q_bits, n_blocks, d_block,
                    sqrt_dim, reference=False, return_levels=False):
    """Scores of the flushed blocks.  q_bits: uint16 [B,1,H,D].  Returns float16
    [B,H,1,(n_blocks+1)*d_block]; positions >= n_blocks*d_block are NaN here (uninitialised in the
    reference, extension/csrc/K_cache.cu:329-333).
    s[b,h,t] = fp16( (sum_d khat[t,d] * q[d]) * half(sqrt_dim) ), extension/csrc/K_cache.cu:206-309.
    """
    q_bits = as_bits(q_bits)
    B, _, H, D = q_bits.shape
    out = np.full((B, H, 1, (n_blocks + 1) * d_block), np.nan, np.float16)
    lv = np.zeros((B, H, D), np.uint8) if reference else k_levels(sum_u8, max_u8)
    if n_blocks > 0:
        hi, mid, last = k_planes_fields(first_8, mid_4, last_4, n_blocks)
        kb = reconstruct(hi, mid, last, lv[:, :, None, :, None])          # [B,H,NB,D,cb]
        kf = as_half(kb).astype(np.float32)
        qf = as_half(q_bits).astype(np.float32).reshape(B, H, D)
        acc = np.einsum("bhzdj,bhd->bhzj", kf, qf, optimize=False).astype(np.float32)
        s = (acc * half_scale(sqrt_dim)).astype(np.float16)
        out[:, :, 0, :n_blocks * d_block] = s.reshape(B, H, n_blocks * d_block)
    return (out, lv) if return_levels else out


def v_cache_test_compute(first_8, test_s_value_bits, test_s_index, top_max_k=TOP_MAX_K):
    """Output-magnitude probe.  test_s_value_bits: uint16 [B,H,1,K]; test_s_index: int32 [B,H,1,K].
    test_o[b,h,d] = fp16( sum_i s_i * |fp16(hi[tok_i,d]<<8 | 0x80)| ), tok_i = idx_i*K + i.
    extension/csrc/V_cache.cu:105-122.
    """
    sv = as_half(as_bits(test_s_value_bits)).astype(np.float32)
    B, H = sv.shape[:2]
    sv = sv.reshape(B, H, top_max_k)
    idx = np.asarray(test_s_index).reshape(B, H, top_max_k).astype(np.int64)
    tok = idx * top_max_k + np.arange(top_max_k)[None, None, :]
    bi = np.arange(B)[:, None, None]
    hi_ = np.arange(H)[None, :, None]
    rows = first_8[bi, hi_, tok]                                           # [B,H,K,D]
    vb = ((rows.astype(np.uint16) << 8) + np.uint16(0x0080)) & np.uint16(0x7FFF)
    vf = as_half(vb).astype(np.float32)
    acc = np.einsum("bhkd,bhk->bhd", vf, sv).astype(np.float32)
    return acc.astype(np.float16).reshape(B, H, 1, -1)


def v_cache_compute(first_8, mid_4, last_4, s_bits, amin_u8, n_tokens, reference=False,
                    return_levels=False):
    """o[b,h,d] = fp16( sum_{t<n_tokens} vhat[t,d] * s[t] ).  s_bits: uint16 [B,H,1,>=n_tokens];
    amin_u8: uint8, first B*H bytes are used (extension/csrc/V_cache.cu:195,337).
    extension/csrc/V_cache.cu:203-307.
    """
    s_bits = as_bits(s_bits)
    B, H = s_bits.shape[:2]
    D = first_8.shape[-1]
    sb = s_bits.reshape(B, H, -1)[:, :, :n_tokens]
    amin = np.asarray(amin_u8, np.uint8).reshape(-1)[:B * H].reshape(B, H)
    lv = np.zeros((B, H, n_tokens), np.uint8) if reference else v_levels(amin, sb)
    if n_tokens == 0:
        o = np.zeros((B, H, 1, D), np.float16)
        return (o, lv) if return_levels else o
    hi, mid, last = v_planes_fields(first_8, mid_4, last_4, n_tokens)
    vb = reconstruct(hi, mid, last, lv[..., None])
    vf = as_half(vb).astype(np.float32)
    sf = as_half(sb).astype(np.float32)
    acc = np.einsum("bhtd,bht->bhd", vf, sf).astype(np.float32)
    o = acc.astype(np.float16).reshape(B, H, 1, D)
    return (o, lv) if return_levels else o


# --------------------------------------------------------------------------------------
# host-side bookkeeping (exponent tracking, probes, thresholds)
# --------------------------------------------------------------------------------------
def colmax_prefill(x_half, literal=True):
    """Column-max exponent at prefill.  x_half: float16 [B,S,H,D] -> uint8 [B,1,H,D].
    literal=True: exponent of the SIGNED maximum over the sequence
    (extension/k_cache_file.py:77-78, extension/v_cache_file.py:80-81);
    literal=False: exponent of the largest magnitude (what the decode update effectively tracks)."""
    x = np.asarray(x_half, np.float16)
    if literal:
        m = x.max(axis=1, keepdims=True)
        return exponent_bits(np.ascontiguousarray(m))
    return exponent_bits(x).max(axis=1, keepdims=True)


def colmax_update(colmax_u8, x_new_half):
    """maximum(colmax, exponent(new token)) -- extension/k_cache_file.py:98-99."""
    return np.maximum(colmax_u8, exponent_bits(np.asarray(x_new_half, np.float16)))


def k_sum_and_max(q_half, k_colmax_u8):
    """q_exp + colmax (uint8) and its max over channels -- extension/k_cache_file.py:136-138."""
    q_exp = exponent_bits(np.asarray(q_half, np.float16))
    s = (q_exp + k_colmax_u8).astype(np.uint8)
    return s, s.max(axis=3, keepdims=True)


def bucket_max(p_half, n_valid, top_max_k=TOP_MAX_K):
    """Arg-max token of every residue class mod top_max_k.
    p_half: float16 [B,H,1,W] (a view of width W of the probabilities).  Mirrors
    V_Cache_Class.test_compute: when W == n_valid the row is zero-padded up to a multiple of
    top_max_k, otherwise the first (W // top_max_k)*top_max_k entries are used; the row is
    viewed as [G, top_max_k] and reduced over G (first maximal index wins).
    extension/v_cache_file.py:121-130.  Returns (values float16 [B,H,1,K], group index int32)."""
    p = np.asarray(p_half, np.float16)
    B, H, _, W = p.shape
    if n_valid == W:
        G = cdiv(n_valid, top_max_k)
        pad = G * top_max_k - W
        if pad:
            p = np.concatenate([p, np.zeros((B, H, 1, pad), np.float16)], axis=-1)
    else:
        G = W // top_max_k
    g = p[..., :G * top_max_k].reshape(B, H, G, top_max_k)
    idx = g.argmax(axis=2)                      # first occurrence of the maximum
    val = np.take_along_axis(g, idx[:, :, None, :], axis=2)
    return val.reshape(B, H, 1, top_max_k), idx.astype(np.int32).reshape(B, H, 1, top_max_k)


def test_o_exponent(test_o_half):
    """`(bits >> 10).to(uint8) & 0x1F - 1` parses as `& 0x1E` -- extension/v_cache_file.py:142."""
    return (exponent_bits(np.asarray(test_o_half, np.float16)) & np.uint8(0x1F - 1)).astype(np.uint8)


def alignment_min(test_o_exp_u8, v_colmax_u8, literal_broadcast=False):
    """amin = min_d (test_o_exp + 15 - v_colmax) in wrapping uint8.
    test_o_exp_u8: [B,H,1,D]; v_colmax_u8: [B,1,H,D].
    literal_broadcast=True reproduces the reference expression as written: the operands
    broadcast to [B,H,H,D], the min is [B,H,H,1] and the kernel reads its first B*H bytes
    (extension/v_cache_file.py:156-160, extension/csrc/V_cache.cu:195,337), i.e. entry f=b*H+h
    pairs the probe of (batch f//H^2, head (f//H)%H) with the column max of head f%H of that batch.
    literal_broadcast=False pairs probe and column max of the same (b,h).  Returns uint8 [B,H]."""
    to = np.asarray(test_o_exp_u8, np.uint8)
    cm = np.asarray(v_colmax_u8, np.uint8)
    B, H, _, D = to.shape
    if literal_broadcast:
        full = (to + np.uint8(FP16_EXP_BIAS) - cm).astype(np.uint8)     # [B,H,H,D]
        mn = full.min(axis=-1)                                          # [B,H,H]
        return np.ascontiguousarray(mn).reshape(-1)[:B * H].reshape(B, H).copy()
    al = (to.reshape(B, H, D) + np.uint8(FP16_EXP_BIAS) - cm.reshape(B, H, D)).astype(np.uint8)
    return al.min(axis=-1)


def softmax_fp32_to_half(scores_half):
    """F.softmax(scores.float(), dim=-1).type_as(q) -- model/KVCache_AlignedKV.py:121."""
    x = np.asarray(scores_half, np.float16).astype(np.float32)
    m = x.max(axis=-1, keepdims=True)
    e = np.exp(x - m, dtype=np.float32)
    return (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float16)


def rest_scores(q_half, restk_half, restlen, head_dim):
    """Scores of the not-yet-flushed tail: fp16 matmul (fp32 accumulate, rounded to fp16) then
    divided by sqrt(D) in fp16 -- extension/k_cache_file.py:156.
    q_half [B,1,H,D], restk_half [B,cb,H,D] -> float16 [B,H,1,restlen]."""
    q = np.asarray(q_half, np.float16).astype(np.float32)[:, 0]                   # [B,H,D]
    k = np.asarray(restk_half, np.float16).astype(np.float32)[:, :restlen]        # [B,r,H,D]
    dot = np.einsum("bhd,brhd->bhr", q, k).astype(np.float32).astype(np.float16)
    s = (dot.astype(np.float32) / np.float32(math.sqrt(head_dim))).astype(np.float16)
    return s[:, :, None, :]


def rest_output(p_half, restv_half, restlen):
    """Tail contribution of the output: fp16 matmul rounded to fp16 -- extension/v_cache_file.py:189.
    p_half [B,H,1,restlen], restv_half [B,cb,H,D] -> float16 [B,H,1,D]."""
    p = np.asarray(p_half, np.float16).astype(np.float32)[:, :, 0]                # [B,H,r]
    v = np.asarray(restv_half, np.float16).astype(np.float32)[:, :restlen]        # [B,r,H,D]
    o = np.einsum("bhr,brhd->bhd", p, v).astype(np.float32).astype(np.float16)
    return o[:, :, None, :]


# --------------------------------------------------------------------------------------
# whole cache + decode step (model/KVCache_AlignedKV.py:72-135 on top of the pieces above)
# --------------------------------------------------------------------------------------
@dataclass
class OracleCache:
    """One layer of K and V state: planes, column-max exponents, fp16 rest buffers.
    extension/k_cache_file.py:14-60, extension/v_cache_file.py:15-63."""
    bsz: int
    max_seq_len: int
    n_heads: int
    head_dim: int
    d_block: int = COLUMN_BLOCK
    k_block: int = COLUMN_BLOCK      # tokens per block of the K planes (a multiple of d_block, the flush unit)
    top_max_k: int = TOP_MAX_K
    literal_colmax: bool = True
    literal_broadcast: bool = False
    reference: bool = False
    cur_len: int = 0
    rest_start: int = 0
    rest_len: int = 0
    k_planes: tuple = field(default=None, repr=False)
    v_planes: tuple = field(default=None, repr=False)
    k_colmax: np.ndarray = field(default=None, repr=False)
    v_colmax: np.ndarray = field(default=None, repr=False)
    restk: np.ndarray = field(default=None, repr=False)
    restv: np.ndarray = field(default=None, repr=False)
    last: dict = field(default_factory=dict, repr=False)   # intermediates of the last decode step

    def __post_init__(self):
        self.k_planes = k_planes_alloc(self.bsz, self.n_heads, self.max_seq_len, self.head_dim, self.k_block)
        self.v_planes = v_planes_alloc(self.bsz, self.n_heads, self.max_seq_len, self.head_dim)
        shp = (self.bsz, 1, self.n_heads, self.head_dim)
        self.k_colmax = np.zeros(shp, np.uint8)
        self.v_colmax = np.zeros(shp, np.uint8)

    # -- save: extension/k_cache_file.py:69-118, extension/v_cache_file.py:72-116 ------
    def save(self, k_half, v_half, start_pos, seqlen):
        cb = self.d_block
        k = np.asarray(k_half, np.float16)
        v = np.asarray(v_half, np.float16)
        assert k.shape == (self.bsz, seqlen, self.n_heads, self.head_dim)
        assert start_pos + seqlen <= self.max_seq_len
        assert start_pos == 0 or seqlen == 1
        assert start_pos == self.cur_len
        self.cur_len += seqlen
        if start_pos == 0:
            self.k_colmax = colmax_prefill(k, self.literal_colmax)
            self.v_colmax = colmax_prefill(v, self.literal_colmax)
            if self.k_block == cb:
                k_cache_save(*self.k_planes, as_bits(k), seqlen // cb, cb, 0, seqlen)
            elif seqlen - seqlen % cb:
                n = seqlen - seqlen % cb      # whole 64-token tiles; the last block may stay partly filled
                k_cache_save(*self.k_planes, as_bits(k[:, :n]), cdiv(n, self.k_block), self.k_block, 0, n)
            v_cache_save(*self.v_planes, as_bits(v), 0, seqlen - seqlen % cb)
            r = seqlen % cb
            self.restk = np.zeros((self.bsz, cb, self.n_heads, self.head_dim), np.float16)
            self.restv = np.zeros_like(self.restk)
            self.restk[:, :r] = k[:, seqlen - r:]
            self.restv[:, :r] = v[:, seqlen - r:]
            self.rest_len = r
            self.rest_start = seqlen - r
        else:
            self.k_colmax = colmax_update(self.k_colmax, k)
            self.v_colmax = colmax_update(self.v_colmax, v)
            self.restk[:, self.rest_len:self.rest_len + 1] = k
            self.restv[:, self.rest_len:self.rest_len + 1] = v
            self.rest_len += 1
            if self.rest_len == cb:
                if self.k_block == cb or self.rest_start == 0:
                    k_cache_save(*self.k_planes, as_bits(self.restk), 1, self.k_block, self.rest_start, cb)
                else:
                    k_cache_save(*self.k_planes, as_bits(self.restk), 1, self.k_block, self.rest_start, cb, tile_append=True)
                v_cache_save(*self.v_planes, as_bits(self.restv), self.rest_start, cb)
                self.rest_len = 0
                self.rest_start += cb
                self.restk = np.zeros_like(self.restk)
                self.restv = np.zeros_like(self.restv)

    # -- decode: model/KVCache_AlignedKV.py:101-124 ----------------------------------------
    def decode(self, q_half, k_half, v_half, mask_half=None):
        """One decode step; q,k,v float16 [B,1,H,D]; mask float16 broadcastable to [B,H,1,L].
        Returns float16 [B,1,H,D]."""
        cb = self.d_block
        B, H, D = self.bsz, self.n_heads, self.head_dim
        start_pos = self.cur_len
        q = np.asarray(q_half, np.float16)
        self.save(k_half, v_half, start_pos, 1)
        L = start_pos + 1
        R = self.rest_start
        nb = cdiv(R, self.k_block)
        # K side: extension/k_cache_file.py:132-159
        ksum, kmax = k_sum_and_max(q, self.k_colmax)
        s, klv = k_cache_compute(*self.k_planes, ksum, kmax, as_bits(q), nb, self.k_block,
                                 1.0 / math.sqrt(D), self.reference, return_levels=True)
        assert self.rest_len + R == L
        if self.rest_len:
            s[:, :, :, R:R + self.rest_len] = rest_scores(q, self.restk, self.rest_len, D)
        s[:, :, :, L:] = -np.inf
        if mask_half is not None:
            s[:, :, :, :L] = (s[:, :, :, :L] + np.asarray(mask_half, np.float16)[..., :L]).astype(np.float16)
        p = softmax_fp32_to_half(s)
        # V side: extension/v_cache_file.py:145-190
        p_cut = p[:, :, :, :R]
        p_test = p_cut if R else p
        tv, ti = bucket_max(p_test, L, self.top_max_k)
        test_o = v_cache_test_compute(self.v_planes[0], as_bits(tv), ti, self.top_max_k)
        to_exp = test_o_exponent(test_o)
        amin = alignment_min(to_exp, self.v_colmax, self.literal_broadcast)
        o, vlv = v_cache_compute(*self.v_planes, as_bits(np.ascontiguousarray(p_cut)) if R else
                                 np.zeros((B, H, 1, 0), np.uint16), amin, R, self.reference,
                                 return_levels=True)
        if self.rest_len:
            o = (o + rest_output(p[:, :, :, R:L], self.restv, self.rest_len)).astype(np.float16)
        self.last = dict(scores=s, probs=p, k_levels=klv, v_levels=vlv, amin=amin, test_o=test_o,
                         test_value=tv, test_index=ti, ksum=ksum, kmax=kmax, R=R, L=L)
        return o.reshape(B, 1, H, D)


def dense_attention(q_half, k_half, v_half, mask_half=None):
    """Dense decode attention with the semantics of model/Llama_AlignedKV.py:130-139:
    fp16 matmul / sqrt(D), + mask, fp32 softmax cast to fp16, fp16 matmul.
    q [B,1,H,D], k/v [B,L,H,D] float16 -> float16 [B,1,H,D]."""
    q = np.asarray(q_half, np.float16).astype(np.float32)[:, 0]
    k = np.asarray(k_half, np.float16).astype(np.float32)
    v = np.asarray(v_half, np.float16).astype(np.float32)
    D = q.shape[-1]
    w = np.einsum("bhd,blhd->bhl", q, k).astype(np.float32).astype(np.float16)
    w = (w.astype(np.float32) / np.float32(math.sqrt(D))).astype(np.float16)
    if mask_half is not None:
        w = (w + np.asarray(mask_half, np.float16).reshape(w.shape[0], -1, w.shape[-1])).astype(np.float16)
    p = softmax_fp32_to_half(w)
    o = np.einsum("bhl,blhd->bhd", p.astype(np.float32), v).astype(np.float32).astype(np.float16)
    return o[:, None]


def algorithmic_bytes(k_levels_bhd, v_levels_bhr, B, H, D, R, L, top_max_k=TOP_MAX_K):
    """Bytes one decode step must move for the given masks, and the dense fp16 figure.
    K planes: R*D*(1 + 1/2 [lvl<2] + 1/2 [lvl==0]) per (b,h) averaged over channels;
    V planes: D*sum_t(1 + 1/2 [lvl<2] + 1/2 [lvl==0]); plus the fp16 tail, q, scores, probe rows."""
    kl = np.asarray(k_levels_bhd)
    vl = np.asarray(v_levels_bhr)
    tail = L - R
    k_plane = float(R) * ((kl >= 0).sum() + 0.5 * (kl < 2).sum() + 0.5 * (kl == 0).sum())
    v_plane = float(D) * ((vl >= 0).sum() + 0.5 * (vl < 2).sum() + 0.5 * (vl == 0).sum())
    k_other = B * H * tail * D * 2 + B * H * D * 3 + B * H + B * H * L * 2
    v_other = B * H * top_max_k * D + B * H * L * 2 + B * H * tail * D * 2 + B * H * D * 2
    dense = 2 * B * H * L * D * 2
    return dict(k_plane=k_plane, v_plane=v_plane, k_total=k_plane + k_other, v_total=v_plane + v_other,
                total=k_plane + v_plane + k_other + v_other, dense=float(dense),
                f_mid_k=float((kl < 2).mean()), f_last_k=float((kl == 0).mean()),
                f_mid_v=float((vl < 2).mean()) if vl.size else 0.0,
                f_last_v=float((vl == 0).mean()) if vl.size else 0.0)
