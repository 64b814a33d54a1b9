// gfx950 (CDNA4, wave64) kernels of the NeuZip bf16 codec.
//
//   nz_split_unpacked_kernel   Manager::split            cuda/high_level.cu:265-321
//   nz_encode_kernel           kernel_aligned_split      cuda/kernels.cuh:62-156
//   nz_encode_long_kernel      + per-chunk exponent histogram, 12-bit frequency
//                              table and its serialized form, then
//                              nvcomp ANS compress       cuda/high_level.cu:103-115
//   nz_compact_kernel          exact-size compaction     cuda/high_level.cu:117-124
//                              (on the device: every record finds its own place)
//   nz_decode_kernel           nvcomp ANS decompress + kernel_aligned_merge fused:
//                              cuda/high_level.cu:184-201, cuda/kernels.cuh:167-217
//
// The whole path is byte/integer work bound by HBM traffic; there is no dense
// contraction, hence no MFMA.  One wavefront decodes one segment with 64
// interleaved rANS states; the exponent never exists in HBM on the decode side.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nz_format.h"

#ifndef NZ_HIST_COPIES
#define NZ_HIST_COPIES 8u
#endif
#define NZ_HIST_STRIDE 257u
#define NZ_RING_WORDS 1024u  // per-wave LDS ring of renormalisation words
#define NZ_RING_DWORDS (NZ_RING_WORDS / 2)

// ----------------------------------------------------------------------------
// element-wise split / merge arithmetic
// ----------------------------------------------------------------------------

// Exponent byte and (sign | kept mantissa) field of one bf16 value.  This is the
// closed form of cuda/kernels.cuh:122-137,153-155: round the 15-bit magnitude
// half-up to S kept mantissa bits, the carry running into the exponent and the
// exponent byte wrapping 255 -> 0 exactly like the reference's uint8 store.
template <int S>
__device__ __forceinline__ void nz_split_one(uint32_t v, uint32_t& exp, uint32_t& repr) {
  if constexpr (S == 7) {
    exp = (v >> 7) & 0xFFu;
    repr = ((v >> 8) & 0x80u) | (v & 0x7Fu);
  } else {
    uint32_t a = ((v & 0x7FFFu) + (1u << (6 - S))) & 0x7FFFu;
    exp = a >> 7;
    repr = ((v >> 15) << S) | ((a >> (7 - S)) & ((1u << S) - 1u));
  }
}

// Position of element j (0..7) of an 8-element group inside the group's S+1
// packed bytes, MSB first (cuda/kernels.cuh:86-89): bit offset inside the
// little-endian integer that holds those bytes.
template <int S>
__device__ __forceinline__ constexpr uint32_t nz_field_shift(int j) {
  return 8u * ((uint32_t)(j * (S + 1)) >> 3) + (7u - S - ((uint32_t)(j * (S + 1)) & 7u));
}

// cuda/kernels.cuh:197-206 for a non-NaN result (the float multiply by +-1.0f of
// :213-216 only moves the sign bit into place).
template <int S>
__device__ __forceinline__ uint32_t nz_merge_one(uint32_t exp, uint32_t repr) {
  uint32_t frac = (repr & ((1u << S) - 1u)) << (7 - S);
  uint32_t sign = (repr >> S) & 1u;
  return (sign << 15) | (exp << 7) | frac;
}

__device__ __forceinline__ float nz_bf16_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
// two floats -> two bf16 in one word, round to nearest even, NaN stays NaN: the
// conversion instruction of gfx950 (v_cvt_pk_bf16_f32)
typedef __bf16 nz_bf16x2 __attribute__((ext_vector_type(2)));
typedef float nz_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t nz_f32_to_bf16x2(float lo, float hi) {
  const nz_f32x2 v = {lo, hi};
  const nz_bf16x2 r = __builtin_convertvector(v, nz_bf16x2);
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t nz_f32_to_bf16(float f) { return nz_f32_to_bf16x2(f, 0.0f) & 0xFFFFu; }

// ----------------------------------------------------------------------------
// block normalizers (cuda/kernels.cuh:94-118 on the split side, :208-216 on the
// merge side): every group of 2^log2n consecutive elements is divided by
// 1.m, m = the 7 mantissa bits of the group's largest magnitude, before the
// split, and multiplied by it again after the merge.  The group stores m << 1
// (the top 8 of the 23 fraction bits of the float 1.m).  Division and product
// run in fp32 and round to bf16, nearest even, and give what the reference's
// float expressions give: the exact quotient A / B of two 8-bit significands
// is never closer to a bf16 rounding boundary (odd / 2^k, k <= 8) than
// 1 / (256 B) > 2^-16 of its value (256 A = odd * B has no solution with
// B < 256), gradual underflow included, so an fp32 quotient that is off by a
// few units in its last place rounds to the same bf16 as the correctly rounded
// one.  The division is therefore a multiplication by the hardware reciprocal
// of 1.m (one unit in the last place).
// ----------------------------------------------------------------------------
struct NzNorm {
  const uint8_t* bytes;  // one per group, null when the tensor is not normalized
  uint32_t log2n;
};

__device__ __forceinline__ float nz_norm_base(uint32_t byte) {
  return __uint_as_float(0x3F800000u | (byte << 15));
}
__device__ __forceinline__ uint32_t nz_norm_div(uint32_t h, uint32_t byte) {
  return nz_f32_to_bf16(nz_bf16_to_f32(h) * __builtin_amdgcn_rcpf(nz_norm_base(byte)));
}
__device__ __forceinline__ uint32_t nz_norm_mul(uint32_t h, uint32_t byte) {
  return nz_f32_to_bf16(nz_bf16_to_f32(h) * nz_norm_base(byte));
}

// The group bytes of the 8 consecutive elements that start at e0 (a multiple of
// 8), one per element: byte j of the result belongs to element e0 + j.  With
// groups of 8 elements or more there is only one, in byte 0.
__device__ __forceinline__ uint64_t nz_norm_load8(const NzNorm& nm, uint64_t e0) {
  if (nm.log2n >= 3) return nm.bytes[e0 >> nm.log2n];
  if (nm.log2n == 0) return *reinterpret_cast<const uint64_t*>(nm.bytes + e0);
  if (nm.log2n == 1) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(nm.bytes + (e0 >> 1));
    return (uint64_t)__builtin_amdgcn_perm(w, w, 0x01010000u) |
           ((uint64_t)__builtin_amdgcn_perm(w, w, 0x03030202u) << 32);
  }
  const uint32_t w = *reinterpret_cast<const uint16_t*>(nm.bytes + (e0 >> 2));
  return (uint64_t)((w & 0xFFu) * 0x01010101u) | ((uint64_t)((w >> 8) * 0x01010101u) << 32);
}

// 8 bf16 values times (MUL) or divided by their group factors; `nb` holds the
// group byte of every element (all the same when a group has 8 elements or more:
// `same`, which saves seven of the eight factor set-ups)
template <bool MUL>
__device__ __forceinline__ uint4 nz_scale8(const uint4 v, const uint64_t nb, const bool same) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t o[4];
  const auto factor = [](uint32_t byte) {
    const float base = nz_norm_base(byte);
    return MUL ? base : __builtin_amdgcn_rcpf(base);
  };
  if (same) {
    const float f = factor((uint32_t)nb & 0xFFu);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float lo = __uint_as_float(w[k] << 16), hi = __uint_as_float(w[k] & 0xFFFF0000u);
      o[k] = nz_f32_to_bf16x2(lo * f, hi * f);
    }
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float f0 = factor((uint32_t)(nb >> (16 * k)) & 0xFFu);
      const float f1 = factor((uint32_t)(nb >> (16 * k + 8)) & 0xFFu);
      const float lo = __uint_as_float(w[k] << 16), hi = __uint_as_float(w[k] & 0xFFFF0000u);
      o[k] = nz_f32_to_bf16x2(lo * f0, hi * f1);
    }
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

#ifndef NZ_TEMPLATES_ONLY
// One byte per group: the mantissa of the largest magnitude (patterns of |x|
// order like the values).  A workgroup covers 2048 elements, a multiple of
// every group size.
__global__ __launch_bounds__(256) void nz_absmax_kernel(const uint16_t* __restrict__ in, uint64_t n,
                                                        uint32_t log2n, uint8_t* __restrict__ norm) {
  __shared__ uint32_t smax[256];
  const uint32_t tid = threadIdx.x;
  const uint64_t blk0 = (uint64_t)blockIdx.x * 2048;
  const uint64_t e0 = blk0 + (uint64_t)tid * 8;
  uint32_t mag[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) mag[j] = 0;
  if (e0 + 8 <= n) {
    const uint4 v = *reinterpret_cast<const uint4*>(in + e0);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) mag[j] = (w[j >> 1] >> (16 * (j & 1))) & 0x7FFFu;
  } else {
    for (uint32_t j = 0; j < 8 && e0 + j < n; ++j) mag[j] = in[e0 + j] & 0x7FFFu;
  }
  if (log2n < 3) {
    const uint32_t gs = 1u << log2n;
    for (uint32_t q = 0; q < 8; q += gs) {
      if (e0 + q >= n) break;
      uint32_t m = 0;
      for (uint32_t j = 0; j < gs; ++j) m = mag[q + j] > m ? mag[q + j] : m;
      norm[(e0 + q) >> log2n] = (uint8_t)((m & 0x7Fu) << 1);
    }
    return;
  }
  uint32_t m8 = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) m8 = mag[j] > m8 ? mag[j] : m8;
  // a group is `per` consecutive threads: butterfly inside the wavefront, then
  // (groups of 1024 elements: two wavefronts) through LDS
  const uint32_t per = 1u << (log2n - 3);
  for (uint32_t o = 1; o < per && o < 64; o <<= 1) {
    const uint32_t other = (uint32_t)__shfl_xor((int)m8, (int)o, 64);
    m8 = other > m8 ? other : m8;
  }
  if (per > 64) {
    if ((tid & 63) == 0) smax[tid >> 6] = m8;
    __syncthreads();
    const uint32_t other = smax[(tid >> 6) ^ 1u];
    m8 = other > m8 ? other : m8;
  }
  if ((tid & (per - 1)) == 0 && e0 < n) norm[e0 >> log2n] = (uint8_t)((m8 & 0x7Fu) << 1);
}

#endif  // NZ_TEMPLATES_ONLY

__device__ __forceinline__ uint32_t nz_lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

__device__ __forceinline__ uint32_t nz_rank_below(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// inclusive prefix sum over the 64 lanes of a wavefront
// Inclusive prefix sum over the 64 lanes with data-parallel-primitive moves:
// four shifted adds inside each row of 16 lanes, then the last lane of row 0
// and 2 is added to rows 1 and 3, and lane 31 to rows 2 and 3.
__device__ __forceinline__ uint32_t nz_wave_scan(uint32_t v, uint32_t lane) {
  (void)lane;
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xF, 0xF, false);  // row_shr:1
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xF, 0xF, false);  // row_shr:2
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xF, 0xF, false);  // row_shr:4
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xF, 0xF, false);  // row_shr:8
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xA, 0xF, false);  // row_bcast:15
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xC, 0xF, false);  // row_bcast:31
  return v;
}
// Sum of a float over the 64 lanes, by the same moves as nz_wave_scan (a fixed
// order of additions); every lane gets the total.
__device__ __forceinline__ float nz_wave_sum(float v) {
#define NZ_DPP_ADD(ctrl, rows)                                                                      \
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, rows, 0xF, false))
  NZ_DPP_ADD(0x111, 0xF);
  NZ_DPP_ADD(0x112, 0xF);
  NZ_DPP_ADD(0x114, 0xF);
  NZ_DPP_ADD(0x118, 0xF);
  NZ_DPP_ADD(0x142, 0xA);
  NZ_DPP_ADD(0x143, 0xC);
#undef NZ_DPP_ADD
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

__device__ __forceinline__ uint32_t nz_get12(const uint8_t* p, uint32_t i) {
  uint32_t bit = 12u * i;
  const uint8_t* q = p + (bit >> 3);
  uint32_t w = (uint32_t)q[0] | ((uint32_t)q[1] << 8);
  return (w >> (bit & 4u)) & 0xFFFu;
}

#ifndef NZ_TEMPLATES_ONLY
// ----------------------------------------------------------------------------
// Manager::split: unpacked exponent and sign|mantissa bytes, precision 7 always
// (cuda/high_level.cu:289-296 forces f_bits_save = 7).
// ----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void nz_split_unpacked_kernel(const uint16_t* __restrict__ in,
                                                                uint64_t n,
                                                                uint8_t* __restrict__ exps,
                                                                uint8_t* __restrict__ fracs,
                                                                const NzNorm nm) {
  uint64_t i0 = ((uint64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i0 >= n) return;
  if (i0 + 8 <= n) {
    uint4 v = *reinterpret_cast<const uint4*>(in + i0);
    if (nm.bytes) v = nz_scale8<false>(v, nz_norm_load8(nm, i0), nm.log2n >= 3);
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint64_t e = 0, f = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t h = (w[j >> 1] >> (16 * (j & 1))) & 0xFFFFu, ex, rp;
      nz_split_one<7>(h, ex, rp);
      e |= (uint64_t)ex << (8 * j);
      f |= (uint64_t)rp << (8 * j);
    }
    *reinterpret_cast<uint64_t*>(exps + i0) = e;
    *reinterpret_cast<uint64_t*>(fracs + i0) = f;
  } else {
    for (uint64_t i = i0; i < n; ++i) {
      uint32_t ex, rp, h = in[i];
      if (nm.bytes) h = nz_norm_div(h, nm.bytes[i >> nm.log2n]);
      nz_split_one<7>(h, ex, rp);
      exps[i] = (uint8_t)ex;
      fracs[i] = (uint8_t)rp;
    }
  }
}

#endif  // NZ_TEMPLATES_ONLY

// ----------------------------------------------------------------------------
// encode: one workgroup per chunk
// ----------------------------------------------------------------------------
//
// Two kernels share the pieces below.  nz_encode_kernel (segments of up to
// NZ_ENC_MAX_LANE_SYMS symbols per lane, which covers every geometry the
// library picks by itself): wavefront k of the workgroup splits segment k of
// the chunk, keeps the exponent bytes of its lanes in registers, and codes
// them from there once the chunk's table exists: the exponents never reach
// memory.  nz_encode_long_kernel (longer segments): all wavefronts split the
// chunk and park the exponents in scratch, then one wavefront per segment
// codes them from there.

#define NZ_ENC_MAX_LANE_SYMS 288u  // 36 groups of 8 symbols per lane: what fits the registers of four wavefronts per SIMD
#define NZ_ENC_LONG_THREADS 1024u

// f(constant I) for I = FROM, FROM + STEP, ... while I < TO (or, with a negative
// step, while I >= TO): straight-line code with compile-time indices, so that
// a register array indexed by I never needs an address
template <int I>
struct NzConst {
  static constexpr int value = I;
};
template <int FROM, int TO, int STEP, class F>
__device__ __forceinline__ void nz_static_for(F&& f) {
  if constexpr ((STEP > 0 && FROM < TO) || (STEP < 0 && FROM >= TO)) {
    f(NzConst<FROM>{});
    nz_static_for<FROM + STEP, TO, STEP>(f);
  }
}

// sums / maxima over the workgroup (at most 16 wavefronts)
__device__ __forceinline__ uint32_t nz_block_sum(uint32_t v, uint32_t* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  uint32_t t = 0;
  for (uint32_t w = 0; w < blockDim.x / 64; ++w) t += red[w];
  return t;
}

__device__ __forceinline__ uint32_t nz_block_max(uint32_t v, uint32_t* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    uint32_t t = __shfl_xor(v, o, 64);
    v = t > v ? t : v;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  uint32_t t = 0;
  for (uint32_t w = 0; w < blockDim.x / 64; ++w) t = red[w] > t ? red[w] : t;
  return t;
}

// LDS of an encode workgroup.  8 histogram copies (one per lane & 7) at a
// stride of 257 words: exponents of weights cluster on a few values, so a
// single copy would serialise most of a wavefront's atomics on one address;
// the odd stride keeps the copies of a bin in different banks.
struct NzEncLds {
  uint32_t hist[NZ_HIST_COPIES * NZ_HIST_STRIDE];
  uint32_t red[16];
  uint32_t scan_s[4];
  uint64_t mw[4];
  uint32_t cf[256];
  // per symbol: x = freq << 20 (renormalisation threshold), y = freq, z = cum,
  // w = bits of a float just below 1 / freq (four units in the last place
  // under the correctly rounded quotient)
  uint4 tab[256];
  uint32_t sbuf[NZ_MAX_SEGS_PER_CHUNK][NZ_STATE_MAX_BYTES / 4];
  uint32_t pad_sym, raw;
  // for records that go straight to their place: the chunk's record sizes, the
  // sum over the chunks before it, whether the wait for those was given up
  uint32_t seg_units[NZ_MAX_SEGS_PER_CHUNK];
  // what the wavefronts found for their segments (words, state bytes) and the table's length, for
  // the thread that sizes the records: the copies in scratch memory are for the kernels that follow
  uint32_t seg_w[NZ_MAX_SEGS_PER_CHUNK], seg_sb[NZ_MAX_SEGS_PER_CHUNK], tab_len;
  uint32_t chunk_total, gave_up;
  uint32_t redo;  // a wavefront ran out of staging room: the chunk is coded again, into the slots
  uint32_t lb[2];  // the two words of the scratch's announcement state, as thread 0 read them
  uint64_t red64[NZ_ENC_LONG_THREADS / 64];
};

// Split one element group: 8 bf16 values -> 8 exponent bytes (byte j of `e` =
// element j) and the S+1 packed bytes (`f`, little-endian).  Two elements at a
// time, both halves of a dword in parallel: the rounding add cannot carry
// from the low half into the high one (0x7FFF + 2^(6-S) < 2^16), so the closed
// form of nz_split_one holds for both halves at once.
template <int S>
__device__ __forceinline__ void nz_split_group(const uint4 v, uint64_t& e, uint64_t& f) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t t[4], p[4];  // per dword: exponents in bytes 0 and 2 | the two (S+1)-bit fields, first element on top
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if constexpr (S == 7) {
      t[k] = (w[k] >> 7) & 0x00FF00FFu;
      p[k] = ((w[k] >> 8) & 0x00800080u) | (w[k] & 0x007F007Fu);  // sign | mantissa in bytes 0 and 2
    } else {
      const uint32_t a = ((w[k] & 0x7FFF7FFFu) + (0x00010001u << (6 - S))) & 0x7FFF7FFFu;
      t[k] = (a >> 7) & 0x00FF00FFu;
      const uint32_t fld = ((w[k] >> (15 - S)) & (0x00010001u << S)) | ((a >> (7 - S)) & (0x00010001u * ((1u << S) - 1u)));
      p[k] = ((fld << (S + 1)) | (fld >> 16)) & ((1u << (2 * S + 2)) - 1u);
    }
  }
  // bytes 0 and 2 of two dwords -> four consecutive bytes
  const uint32_t e_lo = __builtin_amdgcn_perm(t[1], t[0], 0x06040200u), e_hi = __builtin_amdgcn_perm(t[3], t[2], 0x06040200u);
  e = ((uint64_t)e_hi << 32) | e_lo;
  if constexpr (S == 7) {
    const uint32_t f_lo = __builtin_amdgcn_perm(p[1], p[0], 0x06040200u), f_hi = __builtin_amdgcn_perm(p[3], p[2], 0x06040200u);
    f = ((uint64_t)f_hi << 32) | f_lo;
  } else if constexpr (S == 3) {
    f = p[0] | (p[1] << 8) | (p[2] << 16) | (p[3] << 24);  // one byte per pair of elements
  } else if constexpr (S == 1) {
    f = ((p[0] << 4) | p[1]) | (((p[2] << 4) | p[3]) << 8);  // one nibble per pair
  } else {
    f = (p[0] << 6) | (p[1] << 4) | (p[2] << 2) | p[3];      // two bits per pair, element 0 on top
  }
}

template <int S>
__device__ __forceinline__ void nz_store_packed(uint8_t* pp, uint64_t f) {
  if constexpr (S == 7) __builtin_nontemporal_store(f, reinterpret_cast<uint64_t*>(pp));
  else if constexpr (S == 3) __builtin_nontemporal_store((uint32_t)f, reinterpret_cast<uint32_t*>(pp));
  else if constexpr (S == 1) __builtin_nontemporal_store((uint16_t)f, reinterpret_cast<uint16_t*>(pp));
  else __builtin_nontemporal_store((uint8_t)f, pp);
}

// The last elements of the tensor (fewer than 8 in this lane's group): missing
// ones contribute zero bits (cuda/kernels.cuh:92), and only ceil(rem*(S+1)/8)
// packed bytes exist.  -> the exponent bytes, zero above `rem`.
template <int S>
__device__ __forceinline__ uint64_t nz_split_tail(const uint16_t* __restrict__ in, uint64_t gi, uint32_t rem,
                                                  uint8_t* pp, const NzNorm& nm) {
  uint64_t e = 0, f = 0;
  for (uint32_t j = 0; j < rem; ++j) {
    uint32_t h = in[gi + j], ex, rp;
    if (nm.bytes) h = nz_norm_div(h, nm.bytes[(gi + j) >> nm.log2n]);
    nz_split_one<S>(h, ex, rp);
    e |= (uint64_t)ex << (8 * j);
    const uint32_t bit = j * (S + 1);
    f |= (uint64_t)rp << (8u * (bit >> 3) + (7u - S - (bit & 7u)));
  }
  const uint32_t nb = (rem * (S + 1) + 7) / 8;
  for (uint32_t b = 0; b < nb; ++b) pp[b] = (uint8_t)(f >> (8 * b));
  return e;
}

// From the chunk's histogram (cn symbols): the 12-bit frequency table (sum
// exactly 4096), the encoder's per-symbol entries in LDS, the serialized table
// and the chunk record.  Run by the whole workgroup (at least 256 threads).
// -> an estimate of the chunk's coded length in bits (sum of count x -log2 of
// the quantised probability), the same in every thread.
__device__ __forceinline__ uint32_t nz_build_table(NzEncLds& L, const uint32_t cn, uint8_t* __restrict__ out,
                                                   NzChunkInfo* __restrict__ info_c) {
  const uint32_t tid = threadIdx.x;
  // threads 0..255 own one symbol each; the others take part in the reductions
  // with neutral values
  const bool own = tid < 256;
  uint32_t cnt = 0;
  if (own) {
#pragma unroll
    for (uint32_t k = 0; k < NZ_HIST_COPIES; ++k) cnt += L.hist[k * NZ_HIST_STRIDE + tid];
  }
  const uint32_t live = cnt > 0;
  const uint32_t k = nz_block_sum(live, L.red);
  // cnt * (4096 - k) fits 32 bits for chunks of up to 2^19 symbols (every geometry the library
  // chooses itself): a 32-bit division then, a fraction of the 64-bit one's instructions
  uint32_t f = 0;
  if (cn <= (1u << 19)) f = live ? 1u + (cnt * (NZ_M - k)) / cn : 0u;
  else f = live ? 1u + (uint32_t)(((uint64_t)cnt * (NZ_M - k)) / cn) : 0u;
  const uint32_t sum = nz_block_sum(f, L.red);
  // most frequent symbol, lowest index on ties (cnt <= 2^24 fits above the index byte)
  const uint32_t key = nz_block_max(own ? ((cnt << 8) | (255u - tid)) : 0u, L.red);
  const uint32_t imax = 255u - (key & 0xFFu);
  if (tid == imax) f += NZ_M - sum;
  if (k == 1) f = (tid == imax) ? (NZ_M - 1) : ((tid == (imax ^ 1u)) ? 1u : 0u);
  const uint32_t est_bits = nz_block_sum(live ? (uint32_t)((float)cnt * (12.0f - __log2f((float)f))) + 1u : 0u, L.red);

  // exclusive prefix sum over the 256 symbols
  uint32_t incl = f;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    uint32_t t = __shfl_up(incl, o, 64);
    if ((tid & 63) >= (uint32_t)o) incl += t;
  }
  if (own && (tid & 63) == 63) L.scan_s[tid >> 6] = incl;
  __syncthreads();
  if (own) {
    uint32_t woff = 0;
    for (uint32_t w = 0; w < (tid >> 6); ++w) woff += L.scan_s[w];
    const uint32_t cum = woff + incl - f;
    L.tab[tid] = make_uint4(f << 20, f, cum, f ? __float_as_uint(1.0f / (float)f) - 4u : 0u);
  }

  // ---- serialise the table, in parallel ----
  // 256-bit live mask from the ballots of the four owning waves; the rank of a
  // live symbol is the number of live symbols below it.
  const uint64_t bal = __ballot(own && f != 0);
  if (own && (tid & 63) == 0) L.mw[tid >> 6] = bal;
  __syncthreads();
  const uint64_t m0 = L.mw[0], m1 = L.mw[1], m2 = L.mw[2], m3 = L.mw[3];
  const uint32_t kk = (uint32_t)(__popcll(m0) + __popcll(m1) + __popcll(m2) + __popcll(m3));
  if (own && f != 0) {
    const uint32_t w = tid >> 6;
    const uint32_t below = (w > 0 ? (uint32_t)__popcll(m0) : 0u) + (w > 1 ? (uint32_t)__popcll(m1) : 0u) +
                           (w > 2 ? (uint32_t)__popcll(m2) : 0u) +
                           (uint32_t)__popcll(bal & ((1ull << (tid & 63)) - 1ull));
    L.cf[below] = f;
  }
  // a run starts at a live symbol whose predecessor is not live
  const uint64_t s0 = m0 & ~(m0 << 1);
  const uint64_t s1 = m1 & ~((m1 << 1) | (m0 >> 63));
  const uint64_t s2 = m2 & ~((m2 << 1) | (m1 >> 63));
  const uint64_t s3 = m3 & ~((m3 << 1) | (m2 >> 63));
  const uint32_t runs = (uint32_t)(__popcll(s0) + __popcll(s1) + __popcll(s2) + __popcll(s3));
  const bool run_form = runs >= 1 && runs <= NZ_MAX_RUNS;
  const uint32_t head = run_form ? 1u + 2u * runs : 33u;
  __syncthreads();
  // 12-bit fields, two per three bytes
  for (uint32_t pj = tid; 2 * pj < kk; pj += blockDim.x) {
    const uint32_t a = L.cf[2 * pj];
    const bool two = 2 * pj + 1 < kk;
    const uint32_t b = two ? L.cf[2 * pj + 1] : 0u;
    uint8_t* fp = out + head + 3 * pj;
    fp[0] = (uint8_t)(a & 0xFF);
    fp[1] = (uint8_t)((a >> 8) | ((b & 0xF) << 4));
    if (two) fp[2] = (uint8_t)(b >> 4);
  }
  if (!run_form && tid < 32) {
    const uint64_t mq = tid < 8 ? m0 : (tid < 16 ? m1 : (tid < 24 ? m2 : m3));
    out[1 + tid] = (uint8_t)(mq >> (8 * (tid & 7)));
  }
  if (tid == 0) {
    if (run_form) {
      out[0] = (uint8_t)runs;
      const uint64_t mm[4] = {m0, m1, m2, m3};
      const uint64_t ss[4] = {s0, s1, s2, s3};
      uint32_t r = 0;
      for (int w = 0; w < 4; ++w) {
        uint64_t sm = ss[w];
        while (sm) {
          const uint32_t b = (uint32_t)__builtin_ctzll(sm);
          sm &= sm - 1;
          // first symbol at or after the start that is not live
          uint32_t end = 256;
          uint64_t dead = ~mm[w] & ~((b ? (1ull << b) : 1ull) - 1ull);
          if (b == 0) dead = ~mm[w];
          for (int v = w; v < 4; ++v) {
            if (v > w) dead = ~mm[v];
            if (dead) {
              end = 64u * v + (uint32_t)__builtin_ctzll(dead);
              break;
            }
          }
          out[1 + 2 * r] = (uint8_t)(64u * w + b);
          out[2 + 2 * r] = (uint8_t)(end - (64u * w + b) - 1u);
          ++r;
        }
      }
    } else {
      out[0] = NZ_MODE_BITMAP;
    }
    const uint32_t bytes = head + (12 * kk + 7) / 8;
    const uint32_t padded = (bytes + 3) & ~3u;
    for (uint32_t b = bytes; b < padded; ++b) out[b] = 0;
    NzChunkInfo ci;
    ci.tab_len = padded;
    ci.pad_sym = imax;
    ci.raw = 0;
    ci.reserved = 0;
    *info_c = ci;
    L.pad_sym = imax;
    L.tab_len = padded;
  }
  __syncthreads();
  return est_bits;
}

// ----------------------------------------------------------------------------
// per chunk: coded or raw, and the record size of each of its segments (run by one
// thread of the encode kernel once all segments of the chunk are coded)
// ----------------------------------------------------------------------------
__device__ __forceinline__ bool nz_chunk_finalize(uint64_t c, uint64_t n, uint32_t chunk_syms,
                                                  uint32_t seg_syms, uint32_t spc, NzChunkInfo* info,
                                                  const uint32_t* lds_words, const uint32_t* lds_state_bytes,
                                                  uint32_t tab_len, uint32_t* seg_units, uint32_t* chunk_units,
                                                  uint32_t* lds_seg_units, uint32_t* lds_chunk_total) {
  const uint64_t base = c * chunk_syms;
  const uint32_t cn = (uint32_t)((n - base) < chunk_syms ? (n - base) : chunk_syms);
  const uint32_t nseg = (cn + seg_syms - 1) / seg_syms;
  uint64_t rans_total = tab_len, raw_total = 4;
  for (uint32_t k = 0; k < nseg; ++k) {
    const uint32_t sn = (cn - k * seg_syms) < seg_syms ? (cn - k * seg_syms) : seg_syms;
    const uint32_t w = lds_words[k];
    rans_total += lds_state_bytes[k] + 2 * (uint64_t)((w + 1) & ~1u);
    raw_total += ((sn + 3) & ~3u) + (sn == nz_seg_nominal(chunk_syms, seg_syms, spc, k) ? NZ_CARRY_BYTES : 0u);
  }
  const bool raw = rans_total >= raw_total;
  info[c].raw = raw ? 1u : 0u;
  uint32_t chunk_total = 0;  // a record has at most ~2^21 units, a chunk eight records
  for (uint32_t k = 0; k < nseg; ++k) {
    const uint32_t sn = (cn - k * seg_syms) < seg_syms ? (cn - k * seg_syms) : seg_syms;
    const uint32_t w = lds_words[k];
    uint32_t bytes;
    if (raw)
      bytes = (k == 0 ? 4u : 0u) + ((sn + 3) & ~3u) +
              (sn == nz_seg_nominal(chunk_syms, seg_syms, spc, k) ? NZ_CARRY_BYTES : 0u);
    else bytes = (k == 0 ? tab_len : 0u) + lds_state_bytes[k] + 2u * ((w + 1) & ~1u);
    seg_units[c * spc + k] = bytes / 4;
    lds_seg_units[k] = bytes / 4;
    chunk_total += bytes / 4;
  }
  chunk_units[c] = chunk_total;
  *lds_chunk_total = chunk_total;
  return raw;
}

// ----------------------------------------------------------------------------
// rANS encode of one segment by one wavefront
// ----------------------------------------------------------------------------
//
// The 64 lanes run backwards over their symbols.  Per symbol: emit the low 16
// state bits when the state is at or above freq << 20 (ranked into the word
// slot back to front, so that the decoder reads front to back), then
// x = (x / f) << 12 | (x % f) + cum.  A segment's slot holds one word per
// symbol, the most any input can emit, so there is no overflow path; a chunk
// that codes to more than its raw size is stored raw (decided at the end of the
// kernel, once all segments of the chunk are coded).

// the 8 symbols of one group (byte j of `sy` = symbol j), last symbol first
// (words go to the segment's slot in scratch memory, or with LDS to the
// wavefront's staging area: word p of the slot at LDS byte address lds0 + 2 p)
template <bool LDS>
__device__ __forceinline__ void nz_enc_group(uint32_t& x, uint32_t& pos, const uint64_t sy,
                                             const uint4* __restrict__ tab, uint16_t* __restrict__ slot,
                                             const uint32_t lds0) {
  typedef __attribute__((address_space(3))) uint16_t lds_u16;
  // the table entries do not depend on the state: fetch four at a time, up front
#pragma unroll
  for (int h = 1; h >= 0; --h) {
  uint4 e[8];
#pragma unroll
  for (int j = 4 * h; j < 4 * h + 4; ++j) e[j] = tab[(uint32_t)(sy >> (8 * j)) & 0xFFu];
#pragma unroll
  for (int j = 4 * h + 3; j >= 4 * h; --j) {
    const uint32_t f = e[j].y;
    const bool need = x >= e[j].x;
    const uint64_t m = __ballot(need);
    pos -= (uint32_t)__popcll(m);
    if (need) {  // a 32-bit byte offset from the segment's slot: one add-shift for the address
      if constexpr (LDS)
        *(lds_u16*)(uintptr_t)(lds0 + ((pos + nz_rank_below(m)) << 1)) = (uint16_t)(x & 0xFFFFu);
      else
        *reinterpret_cast<uint16_t*>(reinterpret_cast<uint8_t*>(slot) + ((pos + nz_rank_below(m)) << 1)) =
            (uint16_t)(x & 0xFFFFu);
    }
    x = need ? (x >> 16) : x;
    // x < f << 20 here, so the quotient x / f is below 2^20.  The float estimate
    // x * r with r four units in the last place under 1 / f (itself within half
    // a unit) never exceeds the quotient - the roundings of x and of the product
    // add at most one unit each - and falls short of it by less than
    // 2^20 * 11 * 2^-24 < 1: truncated it is the exact quotient or one less,
    // and the remainder tells which.  With the exact quotient q the new state
    // is (q << 12) + (x - q f) + cum = x + q (4096 - f) + cum.
    uint32_t q = (uint32_t)((float)x * __uint_as_float(e[j].w));
    q += (x - __umul24(q, f) >= f) ? 1u : 0u;
    x = __umul24(q, NZ_M - f) + (x + e[j].z);
  }
  }
}

// Final states, variable length: 64 two-bit codes (code c = 5 + c nibbles),
// then the states as a little-endian nibble stream in lane order.  A state
// is >= 2^16, so it takes 20..32 bits; a flat 32 would waste ~4 more per lane.
__device__ __forceinline__ void nz_enc_finish(const uint32_t x, const uint32_t words, const uint64_t seg,
                                              uint32_t* __restrict__ sb, const uint32_t lane,
                                              uint32_t* __restrict__ states, uint32_t* __restrict__ seg_words,
                                              uint32_t* __restrict__ seg_state_bytes, uint32_t* lds_words,
                                              uint32_t* lds_state_bytes) {
  const uint32_t code = (x >> 20 ? 1u : 0u) + (x >> 24 ? 1u : 0u) + (x >> 28 ? 1u : 0u);
  const uint32_t nn = 5u + code;
  const uint32_t incl = nz_wave_scan(nn, lane);
  const uint32_t at = incl - nn;  // nibble offset of this lane's field
  const uint32_t total = __builtin_amdgcn_readlane(incl, 63);
  const uint32_t sbytes = 16u + ((((total + 1u) >> 1) + 3u) & ~3u);
  for (uint32_t i = lane; i < NZ_STATE_MAX_BYTES / 4; i += 64) sb[i] = 0;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  atomicOr(&sb[lane >> 4], code << (2 * (lane & 15)));
  const uint64_t field = (uint64_t)x << (4 * (at & 7));
  atomicOr(&sb[4 + (at >> 3)], (uint32_t)field);
  if (field >> 32) atomicOr(&sb[5 + (at >> 3)], (uint32_t)(field >> 32));
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
  uint32_t* sdst = states + seg * (NZ_STATE_MAX_BYTES / 4);
  for (uint32_t i = lane; i < sbytes / 4; i += 64) sdst[i] = sb[i];
  if (lane == 0) {
    seg_words[seg] = words;
    seg_state_bytes[seg] = sbytes;
    *lds_words = words;
    *lds_state_bytes = sbytes;
  }
}

// The tensors of one encode call ride in the kernel argument block (as the
// items of a decode batch do): the grid of an encode kernel is the
// concatenation of their chunks, that of the scan kernel one workgroup per
// tensor, that of the compaction the concatenation of their segments.
#define NZ_ENC_BATCH_MAX 16
#define NZ_LOOKBACK_ABORT 0xAB0F7EDDu
struct NzEncItem {
  const uint16_t* in;   // dense input
  uint8_t* packed;      // stored sign|mantissa stream
  uint8_t* ws;          // this tensor's slice of the scratch; the offsets below are into it
  uint8_t* comp;        // the container: header, directory, records
  uint64_t comp_cap;    // capacity the container size is checked against
  uint64_t* d_total;    // container size
  uint32_t* d_status;   // bit 0: the container does not fit
  NzNorm nm;            // normalizer bytes (nullptr: none)
  NzGeom g;
  uint64_t exps, tab_ser, info, carry, slots, states, seg_words, seg_sbytes, seg_units, chunk_units;
  uint32_t chunk_end, seg_end;  // running totals over the batch
  // records straight to their place (nz_encode_kernel, `direct` != 0): where the
  // chunks announce their sizes (two words per chunk, offset into ws), the
  // number that marks this call's announcements, how often a chunk looks for
  // an announcement before it gives up, and where it says so (may be null)
  uint64_t pub, nonce;
  uint64_t* d_gave_up;
  uint32_t direct, spin_limit;
  // two words in ws (offset): [0] counts the direct encodes that have used this
  // scratch, advanced by the workgroup of the last chunk - the announcements'
  // mark is made of it and the nonce, so those of an earlier run of the very
  // same call (a replayed graph) do not pass for this run's; [1] holds
  // NZ_LOOKBACK_ABORT after a run in which a workgroup gave up: the next run
  // then leaves the placing to nz_compact_kernel as well (and says so through
  // the same flags) and takes the mark away.  Whatever the memory held
  // before its first use is as good a start as any.
  uint64_t lb_state;
  // `placed`: one byte per segment (offset into ws), left by a direct encode: 1 =
  // the record is in the container and not in the scratch (its words went there
  // from LDS).  nz_compact_kernel with `use_placed` takes such records from
  // `old_comp`, where they lie at the offsets they keep.
  uint64_t placed;
  const uint8_t* old_comp;
  uint32_t use_placed, reserved;
};
struct NzEncBatch {
  uint32_t count;
  uint32_t stage_words;  // nz_encode_kernel: 16-bit words of LDS staging per wavefront (dynamic LDS), 0 = none
  NzEncItem item[NZ_ENC_BATCH_MAX];
};

__device__ __forceinline__ void nz_write_header(uint8_t* comp, const NzGeom& g, uint64_t total) {
  uint32_t* h = reinterpret_cast<uint32_t*>(comp);
  h[0] = NZ_MAGIC;
  h[1] = NZ_FORMAT_VERSION;
  h[2] = (uint32_t)(g.n & 0xFFFFFFFFu);
  h[3] = (uint32_t)(g.n >> 32);
  h[4] = g.chunk_syms;
  h[5] = g.lane_syms;
  h[6] = (uint32_t)g.n_chunks;
  h[7] = (uint32_t)g.n_segs;
  h[8] = (uint32_t)g.dir_off;
  h[9] = (uint32_t)g.rec_off;
  h[10] = (uint32_t)(total & 0xFFFFFFFFu);
  h[11] = (uint32_t)(total >> 32);
  h[12] = h[13] = h[14] = h[15] = 0;
  // the alignment gap between directory and records
  for (uint64_t b = g.dir_off + 4 * (g.n_segs + 1); b < g.rec_off; ++b) comp[b] = 0;
}


// ----------------------------------------------------------------------------
// move a segment record to its final place
// ----------------------------------------------------------------------------
// NT threads (t = 0 .. NT-1) move the record of segment `seg` = segment k of
// chunk c to o0, counted in 4-byte units from the start of the record area
// (`mine` = its size in the same units; ci, sbytes, w: the chunk's info, the
// size of the coder states, the number of words; `words`: where the words are,
// the end of the segment's slot or a staging area in LDS).  With `whole` the
// record is not assembled from its parts but copied from there (the same record
// in another container).  They write the segment's directory entry; those of
// the last segment add the closing entry, the header, the container size and
// the overflow flag.  -> whether the record fits the container (if not, nothing
// of it is written).
template <uint32_t NT>
__device__ __forceinline__ bool nz_move_record(const NzEncItem& it, const uint64_t seg, const uint64_t c,
                                               const uint32_t k, const uint64_t o0, const uint32_t mine,
                                               const NzChunkInfo ci, const uint32_t sbytes, const uint32_t w,
                                               const uint16_t* words, const uint8_t* whole, const uint32_t t) {
  static_assert(NT >= NZ_TAIL_PAD, "too few threads for the closing zeros");
  const NzGeom& g = it.g;
  const uint8_t* __restrict__ tab_ser = it.ws + it.tab_ser;
  const uint8_t* __restrict__ carry = it.ws + it.carry;
  const uint16_t* __restrict__ slots = reinterpret_cast<const uint16_t*>(it.ws + it.slots);
  const uint32_t* __restrict__ states = reinterpret_cast<const uint32_t*>(it.ws + it.states);
  uint8_t* __restrict__ comp = it.comp;
  const uint64_t o1 = o0 + mine;
  const bool fits = o1 <= 0xFFFFFFFFull && g.rec_off + 4 * o1 + NZ_TAIL_PAD <= it.comp_cap;
  if (seg + 1 == g.n_segs && t == 0) {
    const uint64_t total = g.rec_off + 4 * o1 + NZ_TAIL_PAD;
    *it.d_total = total;
    if (!fits) atomicOr(it.d_status, 1u);
  }
  if (!fits) return false;  // (a record before this one may still fit and be written: harmless)
  uint32_t* dir = reinterpret_cast<uint32_t*>(comp + g.dir_off);
  if (t == 0) dir[seg] = (uint32_t)o0;
  uint8_t* dst = comp + g.rec_off + 4 * o0;
  if (seg + 1 == g.n_segs) {
    if (t == 0) {
      dir[g.n_segs] = (uint32_t)o1;
      nz_write_header(comp, g, g.rec_off + 4 * o1 + NZ_TAIL_PAD);
    }
    if (t < NZ_TAIL_PAD) comp[g.rec_off + 4 * o1 + t] = 0;  // closing zeros
  }
  if (whole) {
    if (whole != dst)
      for (uint32_t i = t; i < mine; i += NT)
        reinterpret_cast<uint32_t*>(dst)[i] = reinterpret_cast<const uint32_t*>(whole)[i];
    return true;
  }
  const uint64_t seg_base = c * g.chunk_syms + (uint64_t)k * g.seg_syms;
  const uint32_t nom = nz_seg_nominal(g.chunk_syms, g.seg_syms, g.spc, k);
  const uint32_t sn = (uint32_t)((g.n - seg_base) < nom ? (g.n - seg_base) : nom);
  if (ci.raw) {
    uint32_t off = 0;
    if (k == 0) {
      if (t < 4) dst[t] = t == 0 ? NZ_MODE_RAW : 0;
      off = 4;
    }
    const uint32_t padded = (sn + 3) & ~3u;
    const uint8_t* rawp = reinterpret_cast<const uint8_t*>(slots + seg * g.seg_syms);  // left there by the encode kernel
    for (uint32_t i = t; i < padded; i += NT) dst[off + i] = i < sn ? rawp[i] : 0;
    if (sn == nom)
      for (uint32_t i = t; i < NZ_CARRY_BYTES; i += NT) dst[off + padded + i] = carry[seg * NZ_CARRY_BYTES + i];
    return true;
  }
  uint32_t off = 0;
  if (k == 0) {
    const uint8_t* tb = tab_ser + c * NZ_TABLE_MAX_BYTES;
    for (uint32_t i = t; i < ci.tab_len; i += NT) dst[i] = tb[i];
    off = ci.tab_len;
  }
  uint32_t* sdst = reinterpret_cast<uint32_t*>(dst + off);
  for (uint32_t i = t; i < sbytes / 4; i += NT) sdst[i] = states[seg * (NZ_STATE_MAX_BYTES / 4) + i];
  // the words are 2-byte aligned; they are moved as dwords (two aligned loads and a
  // funnel shift when the source is off by one word; the load past the last word
  // stays inside the scratch buffer or the staging area)
  const uint16_t* src = words;
  const uint32_t mis = (uint32_t)((reinterpret_cast<uintptr_t>(src) >> 1) & 1u);
  const uint32_t* s32 = reinterpret_cast<const uint32_t*>(src - mis);
  uint32_t* wdst = reinterpret_cast<uint32_t*>(dst + off + sbytes);
  const uint32_t nd = (w + 1) / 2;
  const uint32_t nd4 = nd & ~3u;  // four dwords per thread and turn, then the last one to three singly
  for (uint32_t i = 4 * t; i < nd4; i += 4 * NT) {
    const uint32_t a0 = s32[i], a1 = s32[i + 1], a2 = s32[i + 2], a3 = s32[i + 3];
    uint4 v = make_uint4(a0, a1, a2, a3);
    if (mis) {
      const uint32_t a4 = s32[i + 4];
      v = make_uint4(__builtin_amdgcn_alignbit(a1, a0, 16), __builtin_amdgcn_alignbit(a2, a1, 16),
                     __builtin_amdgcn_alignbit(a3, a2, 16), __builtin_amdgcn_alignbit(a4, a3, 16));
    }
    if ((w & 1) && i + 4 == nd) v.w &= 0xFFFFu;  // the padding word of an odd count is zero
    wdst[i] = v.x;
    wdst[i + 1] = v.y;
    wdst[i + 2] = v.z;
    wdst[i + 3] = v.w;
  }
  for (uint32_t i = nd4 + t; i < nd; i += NT) {
    uint32_t v = mis ? __builtin_amdgcn_alignbit(s32[i + 1], s32[i], 16) : s32[i];
    if ((w & 1) && i == nd - 1) v &= 0xFFFFu;
    wdst[i] = v;
  }
  return true;
}

// Segments of up to 8 * NG symbols per lane: the exponents stay in registers.
// Workgroup = max(4, segments per chunk) wavefronts; wavefront k owns segment k.
extern __shared__ uint32_t nz_enc_stage[];  // word staging of nz_encode_kernel: stage_words / 2 dwords per wavefront + 4
#ifdef NZ_PROBE_PHASES
__device__ unsigned long long nz_probe_acc[8];
#define NZ_PROBE_MARK(k)                                        \
  do {                                                          \
    if (threadIdx.x == 0) {                                     \
      const unsigned long long now = __builtin_readcyclecounter(); \
      atomicAdd(&nz_probe_acc[k], now - probe_t);               \
      probe_t = now;                                            \
    }                                                           \
  } while (0)
#else
#define NZ_PROBE_MARK(k)
#endif

template <int S, int NG>
__global__ __launch_bounds__(64 * NZ_MAX_SEGS_PER_CHUNK, 4) void nz_encode_kernel(const NzEncBatch b) {
  __shared__ NzEncLds L;
#ifdef NZ_PROBE_PHASES
  unsigned long long probe_t = __builtin_readcyclecounter();
#endif
  uint32_t t = 0, first = 0;
  while (t + 1 < b.count && blockIdx.x >= b.item[t].chunk_end) {
    first = b.item[t].chunk_end;
    ++t;
  }
  const NzEncItem& it = b.item[t];
  const NzGeom& g = it.g;
  const uint64_t c = blockIdx.x - first;
  const uint64_t n = g.n;
  const uint32_t chunk_syms = g.chunk_syms, seg_syms = g.seg_syms, spc = g.spc;
  const uint16_t* __restrict__ in = it.in;
  const NzNorm nm = it.nm;
  NzChunkInfo* info = reinterpret_cast<NzChunkInfo*>(it.ws + it.info);
  uint32_t* seg_words = reinterpret_cast<uint32_t*>(it.ws + it.seg_words);
  uint32_t* seg_state_bytes = reinterpret_cast<uint32_t*>(it.ws + it.seg_sbytes);
  uint32_t* seg_units = reinterpret_cast<uint32_t*>(it.ws + it.seg_units);

  const uint32_t tid = threadIdx.x;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t lane = tid & 63;
  const uint64_t base = c * chunk_syms;
  const uint32_t cn = (uint32_t)((n - base) < chunk_syms ? (n - base) : chunk_syms);
  const uint64_t seg = c * spc + wave;
  const uint64_t seg_base = base + (uint64_t)wave * seg_syms;
  const bool has_seg = wave < spc && seg_base < n;
  const uint32_t nom = nz_seg_nominal(chunk_syms, seg_syms, spc, wave < spc ? wave : 0u);
  const uint32_t seg_n = has_seg ? (uint32_t)((n - seg_base) < nom ? (n - seg_base) : nom) : 0u;
  const uint32_t ngroups = (seg_n + NZ_GROUP_SYMS - 1) / NZ_GROUP_SYMS;  // at most NG
  const bool seg_full = has_seg && seg_n == nom;

  // State of the scratch's size announcements (see NzEncItem::lb_state): read
  // once, by one thread, long before it is needed, and handed to the others
  // through LDS, so that every thread of the workgroup acts on the same values
  // (another workgroup may change the words while this one starts).
  uint32_t* lb_state = reinterpret_cast<uint32_t*>(it.ws + it.lb_state);
  if (tid == 0) {
    L.lb[0] = it.direct ? __hip_atomic_load(lb_state, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    L.lb[1] = it.direct ? __hip_atomic_load(lb_state + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    L.redo = 0;
  }
  for (uint32_t i = tid; i < NZ_HIST_COPIES * NZ_HIST_STRIDE; i += blockDim.x) L.hist[i] = 0;
  __syncthreads();
  const uint32_t lb_gen = L.lb[0];
  const bool direct = it.direct && L.lb[1] != NZ_LOOKBACK_ABORT;  // this run places its records itself
  uint32_t* myhist = L.hist + (lane & (NZ_HIST_COPIES - 1)) * NZ_HIST_STRIDE;

  // ---- phase 1: split.  Packed bytes go to the stored layout: segment k of a
  // chunk starts at k * seg_keep, and the last NZ_CARRY_BYTES of a full segment
  // go to carry[seg] instead (they ride in the rANS start states).
  const uint32_t seg_keep = seg_syms / 8 * (S + 1) - NZ_CARRY_BYTES;  // of a segment of nominal length
  const uint64_t chunk_keep = (uint64_t)chunk_syms / 8 * (S + 1) - (uint64_t)NZ_CARRY_BYTES * spc;
  const uint32_t keep = nom / 8 * (S + 1) - NZ_CARRY_BYTES;
  uint8_t* pk = it.packed + c * chunk_keep + (uint64_t)wave * seg_keep;
  uint8_t* carry_seg = it.ws + it.carry + seg * NZ_CARRY_BYTES;
  const uint32_t whole = seg_n / NZ_GROUP_SYMS;  // groups in which every lane has 8 elements
  uint64_t ex[NG];
  const auto dest = [&](uint32_t g8) {  // where the packed bytes of this lane's group g8 go
    const uint32_t sb = (g8 * NZ_LANES + lane) * (S + 1);
    return (seg_full && sb >= keep) ? carry_seg + (sb - keep) : pk + sb;
  };
  const auto count8 = [&](uint64_t e) {
#ifndef NZ_PROBE_NO_HIST
#pragma unroll
    for (int j = 0; j < 8; ++j) atomicAdd(&myhist[(uint32_t)(e >> (8 * j)) & 0xFFu], 1u);
#else  // measurement build: the split phase without its histogram (the kernel ends after the phase)
    asm volatile("" ::"v"((uint32_t)e), "v"((uint32_t)(e >> 32)));
#endif
  };
  typedef uint32_t nz_u32x4 __attribute__((ext_vector_type(4)));
  // Four groups at a time, and the loads of the next four are issued before the
  // current four are split: eight 16-byte loads per lane in flight.
  uint4 vn[4];  // the block after the current one
  const auto load4 = [&](uint32_t gv) {
    const uint16_t* src = in + seg_base + (gv * NZ_LANES + lane) * NZ_GROUP;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const nz_u32x4 r = __builtin_nontemporal_load(reinterpret_cast<const nz_u32x4*>(src + q * NZ_GROUP_SYMS));
      vn[q] = make_uint4(r.x, r.y, r.z, r.w);
    }
  };
  if (4 <= whole) load4(0);
  nz_static_for<0, NG, 4>([&](auto g4c) {
    constexpr int g4 = decltype(g4c)::value;
    // the group number as a run-time value for all address arithmetic: with
    // constants the compiler precomputes the addresses of all groups up front
    // and runs out of registers; ex[] keeps its compile-time index
    uint32_t gv = (uint32_t)g4;
    asm volatile("" : "+s"(gv));
    if (gv + 4 <= whole) {
      uint4 v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = vn[q];
      if (gv + 8 <= whole) load4(gv + 4);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (nm.bytes)
          v[q] = nz_scale8<false>(v[q], nz_norm_load8(nm, seg_base + ((gv + q) * NZ_LANES + lane) * NZ_GROUP),
                                  nm.log2n >= 3);
        uint64_t f;
        nz_split_group<S>(v[q], ex[g4 + q], f);
        nz_store_packed<S>(dest(gv + q), f);
        count8(ex[g4 + q]);
      }
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t g8 = gv + q;
        ex[g4 + q] = 0;
        if (g8 < ngroups) {
          const uint32_t idx0 = (g8 * NZ_LANES + lane) * NZ_GROUP;
          const uint64_t gi = seg_base + idx0;
          if (idx0 + 8 <= seg_n) {
            uint4 v = *reinterpret_cast<const uint4*>(in + gi);
            if (nm.bytes) v = nz_scale8<false>(v, nz_norm_load8(nm, gi), nm.log2n >= 3);
            uint64_t f;
            nz_split_group<S>(v, ex[g4 + q], f);
            nz_store_packed<S>(dest(g8), f);
            count8(ex[g4 + q]);
          } else if (idx0 < seg_n) {
            const uint32_t rem = seg_n - idx0;
            ex[g4 + q] = nz_split_tail<S>(in, gi, rem, dest(g8), nm);
            for (uint32_t j = 0; j < rem; ++j) atomicAdd(&myhist[(uint32_t)(ex[g4 + q] >> (8 * j)) & 0xFFu], 1u);
          }
        }
      }
    }
  });
  __threadfence_block();  // the carried bytes are read back below
  __syncthreads();
  NZ_PROBE_MARK(0);
#ifdef NZ_PROBE_NO_HIST
  return;
#endif

  // ---- the chunk's table ----
  const uint32_t est_bits = nz_build_table(L, cn, it.ws + it.tab_ser + c * NZ_TABLE_MAX_BYTES, info + c);
  NZ_PROBE_MARK(1);

  // ---- phase 2: code the segment from the registers, last group first ----
  // The words go to the segment's slot in scratch memory, or, when the records
  // are placed by this kernel and the estimate says they fit, to the wavefront's
  // staging area in LDS (the last `stage_w` words of the slot), from where they
  // are written once, to their final place.  A wavefront that would run out of
  // staging stops; the chunk is then coded again into the slots (the exponents
  // are still in registers).
  const uint32_t cap_words = seg_syms;
  uint16_t* slot = reinterpret_cast<uint16_t*>(it.ws + it.slots) + seg * cap_words;
  const uint32_t stage_w = b.stage_words < cap_words ? b.stage_words : cap_words;
  const uint32_t stage_lo = cap_words - stage_w;  // first word of the slot that has a place in the staging area
  const uint32_t est_seg_words = (uint32_t)(((uint64_t)est_bits * seg_syms / cn) >> 4);
  bool staged = direct && stage_w >= 1024 && est_seg_words + (est_seg_words >> 4) + 64 <= stage_w;
  typedef __attribute__((address_space(3))) uint32_t lds_u32;
  uint32_t* stage = nz_enc_stage + wave * (b.stage_words / 2);
  const uint32_t stage_lds = (uint32_t)(uintptr_t)((lds_u32*)stage);
  uint32_t pos_end = cap_words;  // where the segment's words begin in its slot
  const auto code_segment = [&](auto lds_tag) -> bool {
    constexpr bool LDS = decltype(lds_tag)::value != 0;
    const uint32_t pad = L.pad_sym;
    // a full segment starts from 2^16 | 16 carried bits of the packed stream
    uint32_t x = NZ_L | (seg_full ? (uint32_t)reinterpret_cast<const uint16_t*>(carry_seg)[lane] : 0u);
    uint32_t pos = cap_words;
    bool out_of_room = false;
    nz_static_for<NG - 1, 0, -1>([&](auto g8c) {
      constexpr int g8 = decltype(g8c)::value;
      uint32_t gv = (uint32_t)g8;
      asm volatile("" : "+s"(gv));
      if (gv < ngroups && !out_of_room) {
        if (LDS && pos - stage_lo < NZ_GROUP * NZ_LANES) {  // a group emits at most 512 words
          out_of_room = true;
        } else {
          uint64_t sy = ex[g8];
          if (gv >= whole) {  // the tensor ends inside this group: the most frequent symbol stands in
            const uint32_t idx0 = (gv * NZ_LANES + lane) * NZ_GROUP;
            const uint32_t have = idx0 < seg_n ? seg_n - idx0 : 0u;  // < 8 in some lane
            if (have < 8) {
              const uint64_t keepm = have ? (~0ull >> (64 - 8 * have)) : 0ull;
              sy = (sy & keepm) | ((0x0101010101010101ull * pad) & ~keepm);
            }
          }
          nz_enc_group<LDS>(x, pos, sy, L.tab, slot, stage_lds - 2u * stage_lo);
        }
      }
    });
    if (out_of_room) return true;
    nz_enc_finish(x, cap_words - pos, seg, L.sbuf[wave], lane, reinterpret_cast<uint32_t*>(it.ws + it.states),
                  seg_words, seg_state_bytes, &L.seg_w[wave], &L.seg_sb[wave]);
    pos_end = pos;
    return false;
  };
#pragma nounroll
  for (int pass = 0; pass < 2; ++pass) {
    if (has_seg) {
      if (staged) {
        if (code_segment(NzConst<1>{})) L.redo = 1;
      } else {
        code_segment(NzConst<0>{});
      }
    }
    // every segment of the chunk is coded (or one has run out of staging)
    __threadfence_block();
    __syncthreads();
    if (!(staged && L.redo)) break;
    staged = false;
  }
  NZ_PROBE_MARK(2);
  // decide coded-or-raw and size the records
  if (tid == 0) {
    L.raw = nz_chunk_finalize(c, n, chunk_syms, seg_syms, spc, info, L.seg_w, L.seg_sb, L.tab_len, seg_units,
                              reinterpret_cast<uint32_t*>(it.ws + it.chunk_units), L.seg_units, &L.chunk_total);
    L.gave_up = 0;
  }
  __syncthreads();
  if (L.raw && has_seg) {
    // a chunk that does not compress: its exponent bytes take the place of the words
    uint8_t* rawp = reinterpret_cast<uint8_t*>(slot);
    nz_static_for<0, NG, 1>([&](auto g8c) {
      constexpr int g8 = decltype(g8c)::value;
      uint32_t gv = (uint32_t)g8;
      asm volatile("" : "+s"(gv));
      const uint32_t idx0 = (gv * NZ_LANES + lane) * NZ_GROUP;
      if (idx0 < seg_n) *reinterpret_cast<uint64_t*>(rawp + idx0) = ex[g8];
    });
  }
  if (!it.direct) return;  // the records are placed by nz_compact_kernel
  uint8_t* placed = it.ws + it.placed;  // per segment: its record is in the container and nowhere else
  const bool last_chunk = c + 1 == g.n_chunks;
  if (!direct) {
    // the run before this one ended with a workgroup giving up: nothing is
    // placed, the caller is told, and the mark is taken away for the next run
    if (tid == 0) {
      atomicOr(it.d_status, 4u);
      if (it.d_gave_up) *it.d_gave_up = it.nonce;
      if (last_chunk) {
        __hip_atomic_store(lb_state, lb_gen + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(lb_state + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (has_seg && lane == 0) placed[seg] = 0;
    return;
  }

  // ---- the records go straight to their place ----
  // The chunk announces the size of its records: two words, each with half of
  // the run's 64-bit mark on top and the size (or its complement) below, so
  // that whatever the scratch memory held before cannot pass for an
  // announcement.  Then it adds up the announcements of the chunks before it,
  // waiting for those that are not there yet.  Workgroups of one launch are
  // observed to start in the order of their numbers, so a chunk waited for is
  // normally running or done, and none of them waits before it has announced;
  // nothing guarantees that order across the dies of the device or next to
  // another kernel that fills the compute units, so the wait is bounded
  // (`spin_limit` looks per announcement): a chunk that gives up says so and
  // leaves its records where they are, for nz_compact_kernel.  Nothing but
  // the announcements passes between workgroups: relaxed device-scope
  // accesses, no fences.
  typedef unsigned long long nz_u64;
  nz_u64* pub = reinterpret_cast<nz_u64*>(it.ws + it.pub);  // four words per chunk: size pair, running-total pair
  const uint32_t mark_a = (uint32_t)(it.nonce >> 32) ^ lb_gen, mark_b = (uint32_t)it.nonce ^ (lb_gen * 0x9E3779B1u);
  const uint32_t mark_pa = mark_a ^ 0xA5A5A5A5u, mark_pb = mark_b ^ 0x3C3C3C3Cu;  // a size can never pass for a total
  if (tid == 0) {
    const uint32_t u = L.chunk_total;
    __hip_atomic_store(pub + 4 * c, ((nz_u64)mark_a << 32) | u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(pub + 4 * c + 1, ((nz_u64)mark_b << 32) | (uint32_t)~u, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  }
  NZ_PROBE_MARK(3);
  // The chunks before this one, a window of one per thread at a time, nearest first.  A chunk
  // that has already placed its records has also announced the running total up to and
  // including itself (below); the nearest such chunk ends the walk, so a workgroup reads the
  // announcements of the chunks that ran beside it and one total, not those of every chunk
  // of the tensor.
  uint64_t part = 0;
  bool lost = false;
  if (c <= blockDim.x) {
    // every chunk before this one has a thread of its own: their sizes, nothing else
    if (tid < c) {
      for (uint32_t tries = 0;; ++tries) {
        const nz_u64 a = __hip_atomic_load(pub + 4 * tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const nz_u64 q = __hip_atomic_load(pub + 4 * tid + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((uint32_t)(a >> 32) == mark_a && (uint32_t)(q >> 32) == mark_b && (uint32_t)a == (uint32_t)~(uint32_t)q) {
          part = (uint32_t)a;
          break;
        }
        if (tries >= it.spin_limit) {
          lost = true;
          break;
        }
        __builtin_amdgcn_s_sleep(8);
      }
    }
  } else
  for (uint64_t hi = c; hi > 0;) {
    const uint64_t lo = hi > blockDim.x ? hi - blockDim.x : 0;
    const uint64_t i = lo + tid;
    uint32_t val = 0, key = 0;  // key: position in the window + 1 of an entry that carries a running total
    if (i < hi) {
      for (uint32_t tries = 0;; ++tries) {
        // all four words in flight at once: one round trip per look
        const nz_u64 a = __hip_atomic_load(pub + 4 * i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const nz_u64 q = __hip_atomic_load(pub + 4 * i + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const nz_u64 pa = __hip_atomic_load(pub + 4 * i + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const nz_u64 pq = __hip_atomic_load(pub + 4 * i + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((uint32_t)(pa >> 32) == mark_pa && (uint32_t)(pq >> 32) == mark_pb &&
            (uint32_t)pa == (uint32_t)~(uint32_t)pq) {
          val = (uint32_t)pa;
          key = (uint32_t)(i - lo) + 1u;
          break;
        }
        if ((uint32_t)(a >> 32) == mark_a && (uint32_t)(q >> 32) == mark_b && (uint32_t)a == (uint32_t)~(uint32_t)q) {
          val = (uint32_t)a;
          break;
        }
        if (tries >= it.spin_limit) {
          lost = true;
          break;
        }
        __builtin_amdgcn_s_sleep(8);
      }
    }
    // the same verdict for every thread: did anybody give up, and where is the nearest total
    const uint32_t verdict = nz_block_max(lost ? 0x80000000u : key, L.red);
    if (verdict & 0x80000000u) {
      lost = true;
      break;
    }
    const uint32_t at = (uint32_t)(i - lo) + 1u;  // sizes of the entries after the total, and the total itself
    if (i < hi && (key ? key == verdict : at > verdict)) part += val;
    if (verdict) break;
    hi = lo;
  }
  if (lost) L.gave_up = 1;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) part += __shfl_xor((nz_u64)part, o, 64);
  if (lane == 0) L.red64[wave] = part;
  __threadfence_block();  // also: the raw bytes above are read back by the move
  __syncthreads();
  NZ_PROBE_MARK(4);
  // staged words of this wavefront to their slot, for the kernel that places records afterwards
  const auto unstage = [&]() {
    const uint16_t* sw = reinterpret_cast<const uint16_t*>(stage);
    for (uint32_t p = pos_end + lane; p < cap_words; p += NZ_LANES) slot[p] = sw[p - stage_lo];
  };
  // the workgroup of the last chunk has seen every other announce (or has given
  // up): all of them have read the count, which can now move on
  if (L.gave_up) {
    if (tid == 0) {
      __hip_atomic_store(lb_state + 1, NZ_LOOKBACK_ABORT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      atomicOr(it.d_status, 4u);
      if (it.d_gave_up) *it.d_gave_up = it.nonce;
      if (last_chunk) __hip_atomic_store(lb_state, lb_gen + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (has_seg) {
      if (staged && !L.raw) unstage();
      if (lane == 0) placed[seg] = 0;
    }
    return;
  }
  if (last_chunk && tid == 0)
    __hip_atomic_store(lb_state, lb_gen + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (tid == 0) {
    // the running total up to and including this chunk, for the chunks that come later (32 bits
    // of 4-byte units: a container beyond 16 GiB announces none, and its chunks walk on)
    uint64_t upto = L.chunk_total;
    for (uint32_t q = 0; q < blockDim.x / 64; ++q) upto += L.red64[q];
    if (upto <= 0xFFFFFFFFull) {
      const uint32_t p32 = (uint32_t)upto;
      __hip_atomic_store(pub + 4 * c + 2, ((nz_u64)mark_pa << 32) | p32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(pub + 4 * c + 3, ((nz_u64)mark_pb << 32) | (uint32_t)~p32, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (has_seg) {
    uint64_t o0 = 0;
    for (uint32_t q = 0; q < blockDim.x / 64; ++q) o0 += L.red64[q];
    for (uint32_t q = 0; q < wave; ++q) o0 += L.seg_units[q];
    const bool from_stage = staged && !L.raw;
    const uint16_t* words = from_stage ? reinterpret_cast<const uint16_t*>(stage) + (pos_end - stage_lo) : slot + pos_end;
    NzChunkInfo ci;  // as nz_build_table and nz_chunk_finalize left it in scratch memory, from LDS
    ci.tab_len = L.tab_len;
    ci.pad_sym = L.pad_sym;
    ci.raw = L.raw ? 1u : 0u;
    ci.reserved = 0;
    const bool fits = nz_move_record<64>(it, seg, c, wave, o0, L.seg_units[wave], ci, L.seg_sb[wave],
                                         cap_words - pos_end, words, nullptr, lane);
    if (from_stage && !fits) unstage();
    if (lane == 0) placed[seg] = (from_stage && fits) ? 1 : 0;
  }
  NZ_PROBE_MARK(5);
}

// Longer segments: all wavefronts split the chunk into scratch, then one
// wavefront per segment codes from there.
template <int S>
__global__ __launch_bounds__(NZ_ENC_LONG_THREADS) void nz_encode_long_kernel(const NzEncBatch b) {
  __shared__ NzEncLds L;
  uint32_t t = 0, first = 0;
  while (t + 1 < b.count && blockIdx.x >= b.item[t].chunk_end) {
    first = b.item[t].chunk_end;
    ++t;
  }
  const NzEncItem& it = b.item[t];
  const NzGeom& g = it.g;
  const uint64_t c = blockIdx.x - first;
  const uint64_t n = g.n;
  const uint32_t chunk_syms = g.chunk_syms, seg_syms = g.seg_syms, spc = g.spc;
  const uint16_t* __restrict__ in = it.in;
  const NzNorm nm = it.nm;
  uint8_t* carry = it.ws + it.carry;
  uint8_t* exps = it.ws + it.exps;
  NzChunkInfo* info = reinterpret_cast<NzChunkInfo*>(it.ws + it.info);
  uint32_t* seg_words = reinterpret_cast<uint32_t*>(it.ws + it.seg_words);
  uint32_t* seg_state_bytes = reinterpret_cast<uint32_t*>(it.ws + it.seg_sbytes);
  uint32_t* seg_units = reinterpret_cast<uint32_t*>(it.ws + it.seg_units);

  const uint32_t tid = threadIdx.x;
  const uint64_t base = c * chunk_syms;
  const uint32_t cn = (uint32_t)((n - base) < chunk_syms ? (n - base) : chunk_syms);

  for (uint32_t i = tid; i < NZ_HIST_COPIES * NZ_HIST_STRIDE; i += blockDim.x) L.hist[i] = 0;
  __syncthreads();
  uint32_t* myhist = L.hist + (tid & (NZ_HIST_COPIES - 1)) * NZ_HIST_STRIDE;

  const uint32_t seg_keep = seg_syms / 8 * (S + 1) - NZ_CARRY_BYTES;     // of a segment of nominal length
  const uint64_t chunk_keep = (uint64_t)chunk_syms / 8 * (S + 1) - (uint64_t)NZ_CARRY_BYTES * spc;
  const uint64_t seg0 = c * spc;
  for (uint32_t i = tid * 8; i < cn; i += blockDim.x * 8) {
    const uint64_t gi = base + i;
    const uint32_t sk = i / seg_syms;                       // segment inside the chunk
    const uint32_t sb = (i - sk * seg_syms) / 8 * (S + 1);  // byte inside the segment
    const uint32_t nom = nz_seg_nominal(chunk_syms, seg_syms, spc, sk);
    const uint32_t keep = nom / 8 * (S + 1) - NZ_CARRY_BYTES;
    const bool seg_full = base + (uint64_t)sk * seg_syms + nom <= n;
    uint8_t* pp = (seg_full && sb >= keep) ? carry + (seg0 + sk) * NZ_CARRY_BYTES + (sb - keep)
                                           : it.packed + c * chunk_keep + (uint64_t)sk * seg_keep + sb;
    const uint32_t rem = cn - i;
    uint64_t e;
    if (rem >= 8) {
      uint4 v = *reinterpret_cast<const uint4*>(in + gi);
      if (nm.bytes) v = nz_scale8<false>(v, nz_norm_load8(nm, gi), nm.log2n >= 3);
      uint64_t f;
      nz_split_group<S>(v, e, f);
      nz_store_packed<S>(pp, f);
      *reinterpret_cast<uint64_t*>(exps + gi) = e;
#pragma unroll
      for (int j = 0; j < 8; ++j) atomicAdd(&myhist[(uint32_t)(e >> (8 * j)) & 0xFFu], 1u);
    } else {
      e = nz_split_tail<S>(in, gi, rem, pp, nm);
      for (uint32_t j = 0; j < rem; ++j) {
        exps[gi + j] = (uint8_t)(e >> (8 * j));
        atomicAdd(&myhist[(uint32_t)(e >> (8 * j)) & 0xFFu], 1u);
      }
    }
  }
  __syncthreads();
  nz_build_table(L, cn, it.ws + it.tab_ser + c * NZ_TABLE_MAX_BYTES, info + c);
  // exponents and carried bytes of this chunk are read back below
  __threadfence_block();
  __syncthreads();

  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t lane = tid & 63;
  const uint64_t seg = seg0 + wave;
  const uint64_t seg_base = base + (uint64_t)wave * seg_syms;
  const uint32_t cap_words = seg_syms;
  uint16_t* slot = reinterpret_cast<uint16_t*>(it.ws + it.slots) + seg * cap_words;
  const bool has_seg = wave < spc && seg_base < n;
  uint32_t seg_n = 0;
  if (has_seg) {
    const uint32_t nom = nz_seg_nominal(chunk_syms, seg_syms, spc, wave);
    seg_n = (uint32_t)((n - seg_base) < nom ? (n - seg_base) : nom);
    const uint32_t ngroups = (seg_n + NZ_GROUP_SYMS - 1) / NZ_GROUP_SYMS;
    const uint32_t pad = L.pad_sym;
    const uint8_t* src = exps + seg_base;
    uint32_t x = NZ_L | (seg_n == nom ? (uint32_t)reinterpret_cast<const uint16_t*>(carry)[seg * NZ_LANES + lane] : 0u);
    uint32_t pos = cap_words;
    for (uint32_t gq = ngroups; gq-- > 0;) {
      const uint32_t idx0 = (gq * NZ_LANES + lane) * NZ_GROUP;
      uint64_t sy;
      if (idx0 + 8 <= seg_n) {
        sy = *reinterpret_cast<const uint64_t*>(src + idx0);
      } else {
        sy = 0;
        for (int j = 0; j < 8; ++j) {
          uint32_t bb = (idx0 + j < seg_n) ? src[idx0 + j] : pad;
          sy |= (uint64_t)bb << (8 * j);
        }
      }
      nz_enc_group<false>(x, pos, sy, L.tab, slot, 0u);
    }
    nz_enc_finish(x, cap_words - pos, seg, L.sbuf[wave], lane, reinterpret_cast<uint32_t*>(it.ws + it.states),
                  seg_words, seg_state_bytes, &L.seg_w[wave], &L.seg_sb[wave]);
  }
  __threadfence_block();
  __syncthreads();
  if (tid == 0) L.raw = nz_chunk_finalize(c, n, chunk_syms, seg_syms, spc, info, L.seg_w, L.seg_sb, L.tab_len, seg_units,
                                          reinterpret_cast<uint32_t*>(it.ws + it.chunk_units), L.seg_units,
                                          &L.chunk_total);
  __syncthreads();
  if (L.raw && has_seg) {
    // a chunk that does not compress: its exponent bytes take the place of the words
    uint8_t* rawp = reinterpret_cast<uint8_t*>(slot);
    const uint8_t* src = exps + seg_base;
    for (uint32_t i = lane; i < seg_n; i += 64) rawp[i] = src[i];
  }
}

// ----------------------------------------------------------------------------
// container size, header
// ----------------------------------------------------------------------------

// sum of v over the 256 threads of the workgroup, in every thread
__device__ __forceinline__ uint64_t nz_block_sum64(uint64_t v, uint64_t* red4) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor((unsigned long long)v, o, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red4[threadIdx.x >> 6] = v;
  __syncthreads();
  return red4[0] + red4[1] + red4[2] + red4[3];
}

#ifndef NZ_TEMPLATES_ONLY
// Container size of every tensor of the batch from the record sizes of its
// chunks (one workgroup of 256 threads per tensor): for a caller that wants the
// size before it provides the container's memory.  A tensor without elements
// has no compaction workgroup: its (header-only) container is written here
// when `comp` is known.
__global__ __launch_bounds__(256) void nz_total_kernel(const NzEncBatch b) {
  __shared__ uint64_t red4[4];
  const NzEncItem& it = b.item[blockIdx.x];
  const NzGeom& g = it.g;
  const uint32_t* __restrict__ chunk_units = reinterpret_cast<const uint32_t*>(it.ws + it.chunk_units);
  uint64_t part = 0;
  for (uint64_t i = threadIdx.x; i < g.n_chunks; i += 256) part += chunk_units[i];
  const uint64_t units = nz_block_sum64(part, red4);
  if (threadIdx.x == 0) {
    const uint64_t total = g.rec_off + 4 * units + NZ_TAIL_PAD;
    *it.d_total = total;
    if (total > it.comp_cap || units > 0xFFFFFFFFull) atomicOr(it.d_status, 1u);
    if (g.n_segs == 0 && it.comp && total <= it.comp_cap) {
      nz_write_header(it.comp, g, total);
      reinterpret_cast<uint32_t*>(it.comp + g.dir_off)[0] = 0;
      for (uint32_t q = 0; q < NZ_TAIL_PAD; ++q) it.comp[g.rec_off + q] = 0;
    }
  }
}

// ----------------------------------------------------------------------------
// move every segment record to its final place: one workgroup per segment
// ----------------------------------------------------------------------------
// The workgroup of segment k of chunk c finds where its record goes by itself:
// the record sizes of all chunks before c (one number per chunk, left by the
// encode kernel) plus those of the segments before k in c.
__global__ __launch_bounds__(256) void nz_compact_kernel(const NzEncBatch b) {
  __shared__ uint64_t red4[4];
  uint32_t t = 0, first = 0;
  while (t + 1 < b.count && blockIdx.x >= b.item[t].seg_end) {
    first = b.item[t].seg_end;
    ++t;
  }
  const NzEncItem& it = b.item[t];
  const NzGeom& g = it.g;
  const NzChunkInfo* __restrict__ info = reinterpret_cast<const NzChunkInfo*>(it.ws + it.info);
  const uint32_t* __restrict__ seg_words = reinterpret_cast<const uint32_t*>(it.ws + it.seg_words);
  const uint32_t* __restrict__ seg_state_bytes = reinterpret_cast<const uint32_t*>(it.ws + it.seg_sbytes);
  const uint32_t* __restrict__ seg_units = reinterpret_cast<const uint32_t*>(it.ws + it.seg_units);
  const uint32_t* __restrict__ chunk_units = reinterpret_cast<const uint32_t*>(it.ws + it.chunk_units);
  const uint64_t seg = blockIdx.x - first;
  const uint64_t c = seg / g.spc;
  const uint32_t k = (uint32_t)(seg - c * g.spc);
  const uint32_t tid = threadIdx.x;
  // everything the move depends on is fetched at once: one round of memory latency
  uint64_t part = 0;
  for (uint64_t i = tid; i < c; i += 256) part += chunk_units[i];
  if (tid < k) part += seg_units[c * g.spc + tid];
  const uint32_t mine = seg_units[seg];
  const NzChunkInfo ci = info[c];
  const uint32_t sbytes = seg_state_bytes[seg];
  const uint32_t w = seg_words[seg];
  const bool in_old = it.use_placed && (it.ws + it.placed)[seg] != 0;
  const uint64_t o0 = nz_block_sum64(part, red4);
  const uint16_t* words = reinterpret_cast<const uint16_t*>(it.ws + it.slots) + seg * g.seg_syms + (g.seg_syms - w);
  nz_move_record<256>(it, seg, c, k, o0, mine, ci, sbytes, w, words,
                      in_old ? it.old_comp + g.rec_off + 4 * o0 : nullptr, tid);
}

#endif  // NZ_TEMPLATES_ONLY

// ----------------------------------------------------------------------------
// fused rANS decode + merge: one workgroup per chunk, one wavefront per segment
// ----------------------------------------------------------------------------
//
// LDS: a 4096-entry slot table of 8-byte entries
//          lo = freq | symbol << 24      hi = slot - cum[symbol]
//      (so that one v_mad_u32_u24 of lo's low 24 bits gives the next state and
//      the symbol is a whole byte for v_perm_b32), per wavefront a ring of
//      1024 16-bit units (2 KiB) that is a sliding window over the segment's
//      record (it first holds the record's head: table, coder states, first
//      words), and the 257 cumulative frequencies of the table parse.  Eight
//      wavefronts per chunk need 49 KiB, so three workgroups share the 160 KiB
//      of a CU.
// A rANS step per lane: one table read, one multiply-add, and when the state
// falls below 2^16 a 16-bit word taken at (words consumed so far by the wave +
// rank of the lane among the lanes that need one).

#define NZ_RING_ALLOC_DWORDS NZ_RING_DWORDS
// What the table parse leaves for the slot-table fill (runs, windows, flags)
// lies in the last slots of the table itself; those are filled last, from
// registers.
#define NZ_TMETA_DWORDS (512 + 256 + 4)
#define NZ_TMETA_SLOT ((uint32_t)(NZ_M - 416))  /* first slot under it; a multiple of 32 */
static_assert(2 * (NZ_M - NZ_TMETA_SLOT) >= NZ_TMETA_DWORDS && NZ_TMETA_SLOT % 32 == 0, "parse results fit under the tail");
// dynamic LDS of a decode workgroup whose chunks have up to `spc` segments
#define NZ_DEC_LDS_BYTES(spc) ((size_t)(2 * NZ_M + (spc) * NZ_RING_ALLOC_DWORDS) * 4)

// S+1 packed bytes of one 8-element group, as a little-endian integer
template <int S>
__device__ __forceinline__ uint64_t nz_load_sm(const uint8_t* p) {
  if constexpr (S == 7) return *reinterpret_cast<const uint64_t*>(p);
  else if constexpr (S == 3) return *reinterpret_cast<const uint32_t*>(p);
  else if constexpr (S == 1) return *reinterpret_cast<const uint16_t*>(p);
  else return *p;
}

// 8 decoded values to the dense output as a streaming (non-temporal) 16-byte
// store: for outputs too large to stay in the last-level cache until their
// consumer runs (nz_stream_output).
__device__ __forceinline__ void nz_stream_store(uint16_t* p, const uint4 v) {
  typedef uint32_t nz_u32x4 __attribute__((ext_vector_type(4)));
  const nz_u32x4 q = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(q, reinterpret_cast<nz_u32x4*>(p));
}

// Output policy of a decode.  A tensor whose dense form is at most half of the
// 256 MB last-level cache is written with ordinary stores: the GEMM that
// consumes the weight right after finds it there (decode + matrix-vector
// product of a 128 MiB weight: 66 us instead of 75), and a reused output buffer
// costs nothing extra.  A larger tensor cannot stay resident anyway; writing it
// with streaming stores keeps it from churning the cache (448 MiB: 145 us
// instead of 167).
#ifndef NZ_STREAM_OUT_BYTES
#define NZ_STREAM_OUT_BYTES (128ull << 20)
#endif
NZ_HD static inline bool nz_stream_output(uint64_t n) { return 2 * n > NZ_STREAM_OUT_BYTES; }

// S+1 packed bytes of one group from the stored stream in global memory,
// which a decode reads exactly once: a streaming (non-temporal) load, so that
// the bytes do not displace what the caches could keep.
template <int S>
__device__ __forceinline__ uint64_t nz_stream_sm(const uint8_t* p) {
  if constexpr (S == 7) return __builtin_nontemporal_load(reinterpret_cast<const uint64_t*>(p));
  else if constexpr (S == 3) return __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p));
  else if constexpr (S == 1) return __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(p));
  else return __builtin_nontemporal_load(p);
}

// Merge 8 exponents (byte 3 of ew[j]) with the group's packed bytes into 8
// bf16 values.
template <int S>
__device__ __forceinline__ uint4 nz_merge_group(uint64_t sm, const uint32_t (&ew)[8]) {
  uint32_t o[4];
  if constexpr (S == 7) {
    // out16 = sign << 15 | exp << 7 | mant, byte b = sign << 7 | mant.  Per pair:
    //   t = exponents at bits 7..14 and 23..30 (two v_perm bytes, one shift)
    //   u = bytes [b0 b0 b1 b1]: sign lands on bit 15 / 31, mantissa on 0..6 / 16..22
    //   out = bitfield insert of t's exponent bits into u
    const uint32_t lo = (uint32_t)sm, hi = (uint32_t)(sm >> 32);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t q = __builtin_amdgcn_perm(ew[2 * k + 1], ew[2 * k], 0x0c070c03u);
      const uint32_t t = q << 7;
      const uint32_t w = k < 2 ? lo : hi;
      const uint32_t u = __builtin_amdgcn_perm(0u, w, (k & 1) ? 0x03030202u : 0x01010000u);
      // bitfield insert: (mask & t) | (~mask & u)
      asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(o[k]) : "s"(0x7F807F80u), "v"(t), "v"(u));
    }
  } else {
    // Fewer mantissa bits: the same shape.  A byte that holds an element's sign
    // in bit 7 and its mantissa bits right below goes into both bytes of the
    // element's half (sign on bit 15, mantissa from bit 6 down); what else the
    // byte holds is masked away, and the exponents, alone in their word, are
    // or-ed in.
    const uint32_t lo = (uint32_t)sm;
    constexpr uint32_t keep = 0x80008000u | (((0x7Fu << (7 - S)) & 0x7Fu) * 0x00010001u);
    constexpr int NV = S == 3 ? 2 : (S == 1 ? 4 : 8);
    uint32_t v[NV];  // v[i]: the packed bytes shifted left by i fields
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = lo << (i * (S + 1));
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t q = __builtin_amdgcn_perm(ew[2 * k + 1], ew[2 * k], 0x0c070c03u);
      const uint32_t t = q << 7;
      uint32_t u;
      if constexpr (S == 3) {
        // byte k holds elements 2k (high nibble) and 2k + 1
        u = __builtin_amdgcn_perm(v[1], v[0], (uint32_t)(4 + k) * 0x01010000u + (uint32_t)k * 0x0101u);
      } else if constexpr (S == 1) {
        // byte k / 2 holds elements 4 (k / 2) .. + 3, two bits each
        const uint32_t b = (uint32_t)k >> 1;
        u = __builtin_amdgcn_perm(v[2 * (k & 1) + 1], v[2 * (k & 1)], (4 + b) * 0x01010000u + b * 0x0101u);
      } else {
        // one byte holds the eight signs, element 0 in bit 7
        u = __builtin_amdgcn_perm(v[2 * k + 1], v[2 * k], 0x04040000u);
      }
      o[k] = (u & keep) | t;
    }
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

// ----------------------------------------------------------------------------
// y = W x for one activation row, W decoded on the fly and never written out
// ----------------------------------------------------------------------------
// A group of 512 consecutive weights lies inside one row of W (the row length
// is a multiple of 512), so the row of a group is the same for all lanes.  A
// lane keeps an fp32 partial sum of its 8-element dot products; what happens
// when the wave leaves a row is described at NzGemvWalk.  Row r owns acc[2r]
// (fixed-point sum) and acc[2r + 1] (contribution count in the low half, flag
// in bit 32).
// 40 fraction bits: an absolute resolution of 9e-13 per partial sum; up to 16
// partial sums below 2^18 in magnitude cannot overflow 64 bits.
#define NZ_GEMV_FRAC_BITS 40
#define NZ_GEMV_PART_MAX 262144.0f /* 2^18 */

struct NzGemv {
  const uint16_t* x;      // x_rows activation rows of in_features bf16 values each, 16-byte aligned
  long long* acc;         // two words per row of this tensor and activation row (sum | count and flag), all zero between calls
  uint16_t* y;            // x_rows rows of one bf16 per row of the tensor
  const uint16_t* bias;   // one bf16 per row of the tensor, or null
  uint32_t in_features;   // multiple of 512
  uint32_t x_rows;        // activation rows that exist (1 .. the kernel's MR); the others are neither read nor written
};

// what a lane holds of the activation rows for one group of 8 weights
template <int MR>
struct NzXq {
  uint4 v[MR];
};

typedef __attribute__((ext_vector_type(2))) __bf16 nz_bf16x2;

__device__ __forceinline__ float nz_dot8(const uint4 w, const uint4 x, float acc) {
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(nz_bf16x2, w.x), __builtin_bit_cast(nz_bf16x2, x.x), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(nz_bf16x2, w.y), __builtin_bit_cast(nz_bf16x2, x.y), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(nz_bf16x2, w.z), __builtin_bit_cast(nz_bf16x2, x.z), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(nz_bf16x2, w.w), __builtin_bit_cast(nz_bf16x2, x.w), acc, false);
  return acc;
}

// Position of a wavefront inside W while it walks its segment group by group.
//
// When the wave leaves a row it adds its 64 partial sums in a fixed order.  A row that lies inside the wave's segment is complete then: bias
// added, rounded, stored.  A row shared with other segments goes through the
// row's accumulator pair: the sum in 24.40 fixed point (integer addition is
// associative, so the result does not depend on which wave arrives first; a
// partial sum that is NaN, infinite or beyond 2^18 sets a flag instead and the
// row comes out as NaN), and a counter of contributions; the wave that brings
// the count to the number of segments the row touches converts, stores and
// returns both words to zero.
template <int MR>
struct NzGemvWalk {
  const uint4* xq;     // x as 8-element blocks, already offset by the lane
  NzGemv gv;
  uint64_t row;
  uint64_t seg_first, seg_end;  // elements of the tensor this wave covers
  uint32_t col;        // column of the current group's first element (uniform)
  uint32_t pending;    // groups added since the last flush (uniform)
  uint32_t seg_syms, last_syms, spc, k;  // segment lengths of a chunk, this wave's segment inside it
  uint32_t xstride;    // 16-byte blocks between two activation rows
  uint64_t w_rows;     // rows of the tensor (= elements between two output rows)
  float sum[MR];

  __device__ __forceinline__ void start(const NzGemv& g, const NzGeom& geom, uint64_t first_elem,
                                        uint32_t seg_n, uint32_t wave_in_chunk, uint32_t lane) {
    gv = g;
    xq = reinterpret_cast<const uint4*>(g.x) + lane;
    xstride = g.in_features / NZ_GROUP;
    w_rows = geom.n / g.in_features;
    row = first_elem / g.in_features;
    col = (uint32_t)(first_elem - row * g.in_features);
    seg_first = first_elem;
    seg_end = first_elem + seg_n;
    seg_syms = geom.seg_syms;
    spc = geom.spc;
    last_syms = geom.chunk_syms - (geom.spc - 1) * geom.seg_syms;  // the chunk's (shorter) last segment
    k = wave_in_chunk;
    pending = 0;
#pragma unroll
    for (int m = 0; m < MR; ++m) sum[m] = 0.f;
  }
  __device__ __forceinline__ uint32_t next_col() const {
    return col + NZ_GROUP_SYMS == gv.in_features ? 0u : col + NZ_GROUP_SYMS;
  }
  // the lane's 8 activations of every row for the group at column c (a row that
  // does not exist reads the last one that does)
  __device__ __forceinline__ NzXq<MR> load(uint32_t c) const {
    NzXq<MR> r;
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const uint32_t mm = (uint32_t)m < gv.x_rows ? (uint32_t)m : gv.x_rows - 1u;
      r.v[m] = xq[(uint64_t)mm * xstride + c / NZ_GROUP];
    }
    return r;
  }
  // Segments the row [first, last] touches, this wave's included: walk over the
  // segment boundaries to the left and to the right (a row rarely spans more
  // than two or three segments; no division).
  __device__ __forceinline__ uint32_t segments_of_row(uint64_t first, uint64_t last) const {
    uint32_t count = 1;
    uint64_t at = seg_first;
    uint32_t kk = k;
    while (at > first) {  // the segment before `at` also holds part of the row
      kk = kk ? kk - 1 : spc - 1;
      at -= kk == spc - 1 ? last_syms : seg_syms;
      ++count;
    }
    at = seg_end;
    kk = k;
    while (at <= last) {  // so does the segment that starts at `at`
      kk = kk + 1 == spc ? 0 : kk + 1;
      at += kk == spc - 1 ? last_syms : seg_syms;
      ++count;
    }
    return count;
  }
  __device__ __forceinline__ void store_row(float v, uint32_t m) const {
    if (gv.bias) v += nz_bf16_to_f32(gv.bias[row]);
    gv.y[(uint64_t)m * w_rows + row] = (uint16_t)nz_f32_to_bf16(v);
  }
  __device__ __forceinline__ void flush(uint32_t lane) {
    float t[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) t[m] = nz_wave_sum(sum[m]);
    if (lane == 0) {
      const uint64_t first = row * gv.in_features, last = first + gv.in_features - 1;
      if (first >= seg_first && last < seg_end) {
#pragma unroll
        for (int m = 0; m < MR; ++m)
          if ((uint32_t)m < gv.x_rows) store_row(t[m], (uint32_t)m);
      } else {
        // Device-scope atomics execute at the L2 in the order they are issued by
        // this lane when each one waits for the value the previous returned, so
        // no cache flush is needed: the count is issued only after the sum's old
        // value has come back, the exchanges only after the count's.
        const uint32_t expected = segments_of_row(first, last);
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          if ((uint32_t)m >= gv.x_rows) continue;
          unsigned long long* slot = reinterpret_cast<unsigned long long*>(gv.acc + 2 * (row * MR + m));
          unsigned long long r0;
          if (fabsf(t[m]) < NZ_GEMV_PART_MAX)  // false for NaN as well
            r0 = atomicAdd(slot, (unsigned long long)__float2ll_rn(t[m] * (float)(1ull << NZ_GEMV_FRAC_BITS)));
          else
            r0 = atomicOr(slot + 1, 1ull << 32);
          uint32_t zero;  // 0, but only the hardware knows: ties the next atomic to the returned value
          asm volatile("v_and_b32 %0, 0, %1" : "=v"(zero) : "v"((uint32_t)r0));
          const unsigned long long before = atomicAdd(slot + 1, 1ull + zero);
          if ((uint32_t)before + 1u == expected) {
            const long long a = (long long)atomicExch(slot, 0ull);
            const unsigned long long f = atomicExch(slot + 1, 0ull);
            store_row((f >> 32) ? __uint_as_float(0x7FC00000u)
                                : (float)((double)a * (1.0 / (double)(1ull << NZ_GEMV_FRAC_BITS))),
                      (uint32_t)m);
          }
        }
      }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m) sum[m] = 0.f;
    pending = 0;
  }
  // add the dot products of the current group, then step to the next group
  __device__ __forceinline__ void add(const uint4 w, const NzXq<MR>& x, uint32_t lane) {
#pragma unroll
    for (int m = 0; m < MR; ++m) sum[m] = nz_dot8(w, x.v[m], sum[m]);
    ++pending;
    col = next_col();
    if (col == 0) {
      flush(lane);
      ++row;
    }
  }
};

// Decoder state of one wavefront.
struct NzWaveDec {
  const uint2* lut;
  uint32_t* ring32;       // 512 dwords = 1024 words: a window of the record
  const uint8_t* words;   // start of the record (uniform); word indices count from here
  uint32_t lim;           // largest byte offset from `words` that may be loaded: container end - 16 (uniform)
  uint32_t ring_lds;      // LDS byte address of the ring (the same in all lanes, kept in a vector register)
  uint32_t nwords;        // 16-bit units the record holds, table and states included
  uint32_t lane;
  uint32_t x;             // this lane's rANS state
  uint32_t base;          // words consumed by the wave (the same in all lanes, kept in a vector register)
  uint32_t filled;        // dwords staged into the ring (multiple of 256; uniform)
  uint32_t sel_keep, sel_shift;  // byte selectors of the renormalisation (vector registers)
  uint4 r;                // 8 words per lane fetched during the previous group

  // 16 bytes of the word stream at dword index d (multiple of 4 per lane).
  // Addresses are clamped to the container's closing padding, so every load is
  // unconditional and in bounds; words past the record are never consumed by
  // a valid stream.
  __device__ __forceinline__ uint4 fetch(uint32_t d) const {
    const uint32_t off = 4u * d < lim ? 4u * d : lim;
    const uint32_t* q = reinterpret_cast<const uint32_t*>(words + off);
    return make_uint4(q[0], q[1], q[2], q[3]);
  }

  __device__ __forceinline__ void commit(uint32_t d, const uint4& v) {
    *reinterpret_cast<uint4*>(ring32 + (d & (NZ_RING_DWORDS - 1))) = v;
  }

  // record at comp + pos of a container of comp_bytes (pos + 16 <= comp_bytes)
  __device__ __forceinline__ void attach(const uint8_t* comp, uint64_t comp_bytes, uint64_t pos, uint32_t* ring) {
    typedef __attribute__((address_space(3))) uint32_t lds_u32;
    ring32 = ring;
    ring_lds = (uint32_t)(uintptr_t)((lds_u32*)ring);
    words = comp + pos;
    const uint64_t room = comp_bytes - NZ_TAIL_PAD - pos;
    lim = room < 0xFFFFFFF0ull ? (uint32_t)room : 0xFFFFFFF0u;
  }

  // Stage the first 512 dwords of the record (table of a chunk's first record,
  // coder states, first words) into the ring.
  __device__ __forceinline__ void stage() {
    uint4 v[2];
#pragma unroll
    for (uint32_t q = 0; q < 2; ++q) v[q] = fetch(256 * q + 4 * lane);
#pragma unroll
    for (uint32_t q = 0; q < 2; ++q) commit(256 * q + 4 * lane, v[q]);
    filled = 512;
  }

  // Start decoding from state x0; the words begin `first_word` 16-bit units
  // into the record (at most 348, so at least 676 words are staged ahead).
  __device__ __forceinline__ void start(uint32_t x0, uint32_t first_word) {
    x = x0;
    base = first_word;
    filled = __builtin_amdgcn_readfirstlane(filled);
    r = fetch(filled + 4 * lane);  // the 512 words behind the staged window
    // keep the three per-lane constants in vector registers of their own (an
    // instruction can name only one scalar register or literal)
    sel_keep = 0x07060504u;
    sel_shift = 0x05040100u;
    asm volatile("" : "+v"(sel_keep), "+v"(sel_shift), "+v"(ring_lds), "+v"(base));
  }

  // Decode the next 8 symbols of every lane into byte 3 of ew[0..7].
  //
  // Ring upkeep: the 512 words that follow the staged window wait in
  // registers (`r`, fetched right after the previous commit, addresses clamped
  // to the container); at the start of a group they are committed to the ring
  // if no more than 512 words are still ahead of `base`, and the next 512 are
  // fetched.  A group consumes at most 8 * 64 = 512 words, so at least 512
  // words are ahead at every group start, the window [base, filled) never
  // exceeds the 1024 ring words, and a fetch has at least one group (for
  // exponent data about six) to arrive before its commit.
  //
  // A step issues: slot read, multiply-add, compare, the lane's word index
  // (words consumed by the wave + its rank among the lanes that renormalise:
  // the two mbcnt instructions add the rank to `base`), the index wrapped into
  // the ring, the word read, and one byte permute whose selector either keeps
  // the state or shifts the word in; `base` advances by the ballot's
  // popcount.  No execution-mask changes and three scalar instructions per
  // step (popcount and the two waits).
  __device__ __forceinline__ void group(uint32_t (&ew)[8]) {
    const uint32_t ahead = __builtin_amdgcn_readfirstlane(base);
    if ((2 * filled - ahead) <= 512u) {
      commit(filled + 4 * lane, r);
      filled += 256;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      r = fetch(filled + 4 * lane);
    }
    typedef __attribute__((address_space(3))) const uint16_t lds_cu16;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint2 e = lut[x & (NZ_M - 1)];
      x = __umul24(e.x, x >> NZ_PROB_BITS) + e.y;
      ew[j] = e.x;
      const bool need = x < NZ_L;
      const uint64_t m = __ballot(need);
      const uint32_t widx = __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32),
                                                      __builtin_amdgcn_mbcnt_lo((uint32_t)m, base));
      uint32_t ring_word = widx & (NZ_RING_WORDS - 1);
      asm volatile("" : "+v"(ring_word));  // mask, then one shift-add (not shift, mask, add)
      const uint32_t at = (ring_word << 1) + ring_lds;
      uint32_t w = *(lds_cu16*)(uintptr_t)at;
      // keep the word read unconditional: straight-line code, no exec-mask branch
      asm volatile("" : "+v"(w));
      const uint32_t sel = need ? sel_shift : sel_keep;
      x = __builtin_amdgcn_perm(x, w, sel);  // x << 16 | w where the state fell below 2^16
      base += (uint32_t)__popcll(m);
    }
  }
};

// One workgroup decodes chunk `c` of one tensor; wavefront k of the workgroup
// takes segment k of the chunk (wavefronts beyond the chunk's segments only
// help to build the slot table).
// With GEMV the decoded values are not stored: they are multiplied with the
// activation `gv.x` and summed into `gv.acc` (the tensor is a row-major matrix
// with rows of gv.in_features elements, a multiple of 512, so that no group is
// ragged and no group straddles two rows).
// With NORM every merged value is multiplied by its group's factor (`nm`)
// before it is stored or used.
template <int S, int GEMV, bool NORM, bool STREAM>
__device__ __forceinline__ void nz_decode_chunk(
    const uint8_t* __restrict__ comp, const uint64_t comp_bytes, const uint8_t* __restrict__ packed,
    uint16_t* __restrict__ out, const NzGeom& g, uint32_t* __restrict__ d_status, const uint64_t c,
    const NzGemv& gv, const NzNorm& nm) {
  extern __shared__ uint32_t lds[];
  uint2* lut = reinterpret_cast<uint2*>(lds);                   // 4096 x 8 bytes
  uint32_t* rings = lds + 2 * NZ_M;                             // spc rings
  uint32_t* tmeta = lds + 2 * NZ_TMETA_SLOT;                    // what the table parse leaves for the fill:
  uint2* runs = reinterpret_cast<uint2*>(tmeta);                //   per live symbol (freq | symbol << 24, first slot)
  uint2* wins = runs + 256;                                     //   per 32 slots (bitmap of run starts, runs before)
  uint32_t* tflag = reinterpret_cast<uint32_t*>(wins + 128);    //   [0] frequencies sum to 4096, [1] table bytes
  const uint8_t* tb = reinterpret_cast<const uint8_t*>(rings);  // table bytes: start of the first record

  const uint32_t tid = threadIdx.x;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: keep it scalar
  const uint32_t lane = tid & 63;
  const uint64_t seg0 = c * g.spc;
  const uint64_t chunk_base = c * g.chunk_syms;
  const uint32_t cn =
      (uint32_t)((g.n - chunk_base) < g.chunk_syms ? (g.n - chunk_base) : g.chunk_syms);
  const uint32_t nseg = (cn + g.seg_syms - 1) / g.seg_syms;
  const uint32_t* dir = reinterpret_cast<const uint32_t*>(comp + g.dir_off);

  // the container must be the one the caller's geometry describes
  if (c == 0 && tid == 0) {
    const uint32_t* h = reinterpret_cast<const uint32_t*>(comp);
    if (h[0] != NZ_MAGIC || h[1] != NZ_FORMAT_VERSION || h[2] != (uint32_t)g.n || h[3] != (uint32_t)(g.n >> 32) ||
        h[4] != g.chunk_syms || h[5] != g.lane_syms)
      atomicOr(d_status, 16u);
  }

  // Two rounds of global loads, then only LDS: every wavefront reads the
  // chunk's directory entries itself, then stages the first 2 KiB of its
  // record into its ring (for the chunk's first record that window begins with
  // the table, which all wavefronts parse from there) and fetches the packed
  // bytes of its first group.
  const uint32_t dv = lane <= nseg ? dir[seg0 + lane] : 0u;
  const uint64_t f0 = __builtin_amdgcn_readlane(dv, 0), f1 = __builtin_amdgcn_readlane(dv, 1);
  if (f1 <= f0 || g.rec_off + 4 * f1 + NZ_TAIL_PAD > comp_bytes) {
    if (tid == 0) atomicOr(d_status, 2u);
    return;
  }
  const bool has_seg = wave < nseg;
  const uint32_t wk = has_seg ? wave : 0u;  // wavefronts without a segment only help with the table
  const uint64_t seg_base = chunk_base + (uint64_t)wk * g.seg_syms;
  const uint32_t nom = nz_seg_nominal(g.chunk_syms, g.seg_syms, g.spc, wk);
  const uint32_t seg_n = (uint32_t)((g.n - seg_base) < nom ? (g.n - seg_base) : nom);
  const uint32_t ngroups = (seg_n + NZ_GROUP_SYMS - 1) / NZ_GROUP_SYMS;
  const uint64_t o0 = __builtin_amdgcn_readlane(dv, wk), o1 = __builtin_amdgcn_readlane(dv, wk + 1);
  const bool bad_rec = o1 < o0 || g.rec_off + 4 * o1 + NZ_TAIL_PAD > comp_bytes;
  const uint64_t rec_pos = g.rec_off + 4 * o0;  // uniform: the readlanes above are scalar
  const uint32_t rec_all = (uint32_t)(4 * (o1 - o0));
  // stored packed layout: every full segment keeps seg_p - 128 bytes, its last
  // 128 bytes ride in the coder states (or behind the symbols of a raw record)
  const bool carry = seg_n == nom;
  const uint32_t keep = nom / 8 * (S + 1) - NZ_CARRY_BYTES;
  const uint64_t chunk_keep = (uint64_t)g.chunk_syms / 8 * (S + 1) - (uint64_t)NZ_CARRY_BYTES * g.spc;
  const uint8_t* pk = packed + c * chunk_keep + (uint64_t)wk * (g.seg_syms / 8 * (S + 1) - NZ_CARRY_BYTES);
  uint16_t* dst = out + seg_base;
  // groups whose packed bytes are (partly) carried are merged after the loop
  const uint32_t tailg = carry ? (S == 0 ? 2u : 1u) : 0u;
  const uint32_t body = ngroups - tailg;
  // Groups in which every lane has 8 elements run without any predicate; the
  // packed bytes are fetched one group ahead of their use (the address of the
  // fetch past the last group is clamped, its value unused).
  const uint32_t whole = seg_n / NZ_GROUP_SYMS < body ? seg_n / NZ_GROUP_SYMS : body;
  const uint32_t lane_off = lane * (S + 1);
  const uint32_t last_off = whole ? (whole - 1) * NZ_LANES * (S + 1) + lane_off : 0u;
  NzWaveDec w;
  w.lut = lut;
  w.attach(comp, comp_bytes, bad_rec ? 0 : rec_pos, rings + wk * NZ_RING_ALLOC_DWORDS);
  w.nwords = rec_all / 2;
  w.lane = lane;
  w.filled = 0;
  uint64_t sm_next = 0, nb_next = 0;
  constexpr int MR = GEMV ? GEMV : 1;  // activation rows a lane multiplies with (GEMV: 0 = plain decode)
  // the activations of the next group are fetched a group ahead, unless that would cost the
  // registers of a whole workgroup per compute unit (eight rows: 32 registers)
  constexpr bool X_AHEAD = MR < 8;
  NzXq<X_AHEAD ? MR : 1> xq_next{};
  NzGemvWalk<MR> walk;
  if (has_seg && !bad_rec) {
    w.stage();
    if constexpr (GEMV) {
      walk.start(gv, g, seg_base, seg_n, wk, lane);
      if constexpr (X_AHEAD) xq_next = walk.load(walk.col);
    }
    if (whole) {
      sm_next = nz_stream_sm<S>(pk + lane_off);
      if constexpr (NORM) nb_next = nz_norm_load8(nm, seg_base + lane * NZ_GROUP);
    }
  }
  __syncthreads();
  // the first 32 table bytes hold the mode and all run descriptors there can be
  const uint4 h0 = reinterpret_cast<const uint4*>(tb)[0], h1 = reinterpret_cast<const uint4*>(tb)[1];
  const uint32_t bm_byte = tb[1 + (lane >> 1)];  // bitmap mode: the byte with this lane's four symbols
  const uint32_t mode = h0.x & 0xFFu;
  uint32_t tab_len = 4;

  if (mode != NZ_MODE_RAW) {
    if (mode > NZ_MAX_RUNS) {
      if (tid == 0) atomicOr(d_status, 2u);
      return;
    }
    // Wavefront 0 parses the table, four symbols per lane, and leaves for the
    // fill below: the live symbols in order (`runs`: frequency, symbol, first
    // slot) and, per window of 32 slots, which slots start a run and how many
    // runs start before the window (`wins`).
    if (wave == 0) {
      wins[lane] = make_uint2(0u, 0u);
      wins[lane + 64] = make_uint2(0u, 0u);
      uint32_t head, kk = 0, live4 = 0;
      uint32_t rk[4] = {0, 0, 0, 0};  // rank of the symbol among those the table lists
      if (mode == NZ_MODE_BITMAP) {
        head = 33;
        live4 = (bm_byte >> (4 * (lane & 1))) & 15u;
        const uint32_t c = (uint32_t)__popc(live4);
        const uint32_t ci = nz_wave_scan(c, lane);
        kk = __builtin_amdgcn_readlane(ci, 63);
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) rk[j] = ci - c + (uint32_t)__popc(live4 & ((1u << j) - 1u));
      } else {
        head = 1 + 2 * mode;
        const uint32_t hw[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
        uint32_t acc = 0;
#pragma unroll
        for (uint32_t r = 0; r < NZ_MAX_RUNS; ++r) {
          if (r < mode) {
            const uint32_t st = (hw[(1 + 2 * r) >> 2] >> (8 * ((1 + 2 * r) & 3))) & 0xFFu;
            const uint32_t ln = ((hw[(2 + 2 * r) >> 2] >> (8 * ((2 + 2 * r) & 3))) & 0xFFu) + 1u;
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
              const uint32_t sym = 4 * lane + j;
              if (sym >= st && sym < st + ln) {
                live4 |= 1u << j;
                rk[j] = acc + sym - st;
              }
            }
            acc += ln;
          }
        }
        kk = acc;
      }
      if (kk > 256) kk = 256;  // corrupt input: stay inside the staged bytes
      uint32_t fr[4], tot = 0, nz4 = 0;
#pragma unroll
      for (uint32_t j = 0; j < 4; ++j) {
        const uint32_t f = nz_get12(tb + head, rk[j] > 255 ? 255u : rk[j]);  // read in any case: no branch
        fr[j] = ((live4 >> j) & 1u) ? f : 0u;
        tot += fr[j];
        nz4 += fr[j] ? 1u : 0u;
      }
      // one scan for both the cumulative frequency (below 2^20) and the number of
      // symbols with a nonzero frequency (from bit 20 up)
      const uint32_t mine = tot | (nz4 << 20);
      const uint32_t incl = nz_wave_scan(mine, lane);
      const uint32_t all = __builtin_amdgcn_readlane(incl, 63);
      const bool sums = (all & 0xFFFFFu) == NZ_M;
      if (lane == 0) {
        tflag[0] = sums ? 1u : 0u;
        tflag[1] = (head + (12 * kk + 7) / 8 + 3) & ~3u;
      }
      if (sums) {  // only then do the first slots stay below 4096
        uint32_t first = (incl - mine) & 0xFFFFFu, k = (incl - mine) >> 20;
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
          if (fr[j]) {
            runs[k] = make_uint2(fr[j] | ((4 * lane + j) << 24), first);
            atomicOr(&wins[first >> 5].x, 1u << (first & 31));
            ++k;
            first += fr[j];
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        // runs that start before each window: prefix of the bitmap's popcounts
        const uint32_t b0 = wins[2 * lane].x, b1 = wins[2 * lane + 1].x;
        const uint32_t c0 = (uint32_t)__popc(b0), c1 = (uint32_t)__popc(b1);
        const uint32_t pi = nz_wave_scan(c0 + c1, lane);
        wins[2 * lane].y = pi - c0 - c1;
        wins[2 * lane + 1].y = pi - c1;
      }
    }
    __syncthreads();
    // slot table: consecutive threads fill consecutive slots.  The run of a
    // slot is the number of runs that start at or before it, minus one.  (Of a
    // table whose frequencies do not sum to 4096 nothing was written: the fill
    // then reads zeros and the chunk is given up right after.)  The last slots
    // lie under the parse results: their entries wait in registers until every
    // thread has read what it needs.
    {
      const uint32_t below = (2u << (tid & 31)) - 1u;  // bits of a window up to this thread's slot
      const auto entry_of = [&](uint32_t slot) {
        const uint2 wn = wins[slot >> 5];
        const uint32_t k = wn.y + (uint32_t)__popc(wn.x & below) - 1u;
        const uint2 rn = runs[k & 255u];
        return make_uint2(rn.x, slot - rn.y);
      };
      for (uint32_t slot = tid; slot < NZ_TMETA_SLOT; slot += blockDim.x) lut[slot] = entry_of(slot);
      // (NZ_TMETA_SLOT is a multiple of 32, so `below` fits these slots as well)
      constexpr uint32_t LAST = (NZ_M - NZ_TMETA_SLOT + 63) / 64;  // per thread, for the smallest workgroup
      uint2 last[LAST];
#pragma unroll
      for (uint32_t i = 0; i < LAST; ++i) {
        const uint32_t slot = NZ_TMETA_SLOT + tid + i * blockDim.x;
        last[i] = slot < NZ_M ? entry_of(slot) : make_uint2(0u, 0u);
      }
      const uint32_t table_ok = tflag[0], table_len = tflag[1];
      __syncthreads();
#pragma unroll
      for (uint32_t i = 0; i < LAST; ++i) {
        const uint32_t slot = NZ_TMETA_SLOT + tid + i * blockDim.x;
        if (slot < NZ_M) lut[slot] = last[i];
      }
      if (!table_ok) {
        if (tid == 0) atomicOr(d_status, 2u);
        return;
      }
      tab_len = table_len;
    }
  }
  __syncthreads();

  if (!has_seg) return;
  if (bad_rec) {
    if (lane == 0) atomicOr(d_status, 2u);
    return;
  }
  // the chunk's first record begins with the table
  const uint32_t rec_skip = wave == 0 ? tab_len : 0u;
  if (rec_all < rec_skip) {
    if (lane == 0) atomicOr(d_status, 2u);
    return;
  }
  const uint64_t rec_start = rec_pos + rec_skip;
  const uint32_t rec_bytes = rec_all - rec_skip;

  if (mode == NZ_MODE_RAW) {
    const uint32_t padded = (seg_n + 3) & ~3u;
    if (rec_bytes < padded + (carry ? NZ_CARRY_BYTES : 0u)) {
      if (lane == 0) atomicOr(d_status, 2u);
      return;
    }
    const uint8_t* raw = comp + rec_start;
    const uint8_t* tailp = raw + padded;
    for (uint32_t gq = 0; gq < ngroups; ++gq) {
      const uint32_t idx0 = (gq * NZ_LANES + lane) * NZ_GROUP;
      if (idx0 >= seg_n) continue;
      const uint32_t rem = seg_n - idx0;
      const uint32_t b = idx0 / 8 * (S + 1);
      if (rem >= 8) {
        uint64_t sy = (uint64_t)reinterpret_cast<const uint32_t*>(raw + idx0)[0] |
                      ((uint64_t)reinterpret_cast<const uint32_t*>(raw + idx0)[1] << 32);
        const uint64_t sm = (carry && b >= keep) ? nz_load_sm<S>(tailp + (b - keep)) : nz_load_sm<S>(pk + b);
        uint32_t ew[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) ew[j] = (uint32_t)((sy >> (8 * j)) & 0xFFu) << 24;
        uint4 mv = nz_merge_group<S>(sm, ew);
        if constexpr (NORM) mv = nz_scale8<true>(mv, nz_norm_load8(nm, seg_base + idx0), nm.log2n >= 3);
        if constexpr (GEMV) walk.add(mv, walk.load(walk.col), lane);
        else *reinterpret_cast<uint4*>(dst + idx0) = mv;
      } else if constexpr (!GEMV) {
        for (uint32_t j = 0; j < rem; ++j) {
          const uint32_t bit = (idx0 + j) * (S + 1);
          const uint32_t rp = ((uint32_t)pk[bit >> 3] >> (7u - S - (bit & 7u))) & ((2u << S) - 1u);
          uint32_t h = nz_merge_one<S>(raw[idx0 + j], rp);
          if constexpr (NORM) h = nz_norm_mul(h, nm.bytes[(seg_base + idx0 + j) >> nm.log2n]);
          dst[idx0 + j] = (uint16_t)h;
        }
      }
    }
    if constexpr (GEMV)
      if (walk.pending) walk.flush(lane);
    return;
  }

  if (rec_bytes < 16) {
    if (lane == 0) atomicOr(d_status, 2u);
    return;
  }
  // final encoder states, read from the staged window: 64 two-bit length
  // codes, then a nibble stream
  const uint32_t* rec32 = w.ring32 + rec_skip / 4;
  const uint32_t nn = 5u + ((rec32[lane >> 4] >> (2 * (lane & 15))) & 3u);
  const uint32_t incl = nz_wave_scan(nn, lane);
  const uint32_t at = incl - nn;
  const uint32_t sbytes = 16u + ((((__builtin_amdgcn_readlane(incl, 63) + 1u) >> 1) + 3u) & ~3u);
  if (rec_bytes < sbytes) {
    if (lane == 0) atomicOr(d_status, 2u);
    return;
  }
  // the 8 bytes read here may reach into the words: still inside the window
  const uint32_t fb = 16u + (at >> 1);
  const uint64_t win = (uint64_t)rec32[fb >> 2] | ((uint64_t)rec32[(fb >> 2) + 1] << 32);
  const uint32_t x0 = (uint32_t)(win >> (8 * (fb & 3) + 4 * (at & 1))) & (0xFFFFFFFFu >> (32 - 4 * nn));
  w.start(x0, (rec_skip + sbytes) / 2);

  // Groups in which every lane has 8 elements.  Packed bytes (and normalizer
  // bytes) are fetched TWO groups before their use, alternately into two
  // registers, so that the wait in front of a merge is for a load issued two
  // groups (about two microseconds) earlier and for nothing younger: neither
  // the latency of a load that misses every cache nor the previous group's
  // store is waited for.
  const auto sm_at = [&](uint32_t gq) {
    const uint32_t off = gq * NZ_LANES * (S + 1) + lane_off;
    return nz_stream_sm<S>(pk + (off < last_off ? off : last_off));
  };
  // `wide`: groups of 8 elements or more, one byte per lane and group.  The
  // walk over the full groups exists once per case, so that the common one has
  // no branch between the byte's load and its use two groups later (a load
  // behind a branch is waited for at the join, with every store before it).
  const auto nb_at = [&](uint32_t gq, auto wide) -> uint64_t {
    const uint64_t e0 = seg_base + ((gq < whole ? gq : whole - 1) * NZ_LANES + lane) * NZ_GROUP;
    if constexpr (decltype(wide)::value) return nm.bytes[e0 >> nm.log2n];
    else return nz_norm_load8(nm, e0);
  };
  const auto full_group = [&](uint32_t gq, const uint64_t sm, const uint64_t nb, auto wide) {
    NzXq<MR> xq;
    if constexpr (GEMV && X_AHEAD) {
      xq = xq_next;
      xq_next = walk.load(walk.next_col());  // always inside x
    } else if constexpr (GEMV) {
      xq = walk.load(walk.col);
    }
    uint32_t ew[8];
    w.group(ew);
    // the merge starts only here: its wait for the packed bytes must not be
    // hoisted in front of the rANS steps
    uint32_t sml = (uint32_t)sm, smh = (uint32_t)(sm >> 32);
    asm volatile("" : "+v"(sml), "+v"(smh), "+v"(ew[7]));
    uint4 mv = nz_merge_group<S>(((uint64_t)smh << 32) | sml, ew);
    if constexpr (NORM) mv = nz_scale8<true>(mv, nb, decltype(wide)::value);
    if constexpr (GEMV) walk.add(mv, xq, lane);
    else if constexpr (STREAM) nz_stream_store(dst + (gq * NZ_LANES + lane) * NZ_GROUP, mv);
    else *reinterpret_cast<uint4*>(dst + (gq * NZ_LANES + lane) * NZ_GROUP) = mv;
  };
  const auto full_groups = [&](auto wide) {
    uint64_t sm_a = sm_next, sm_b = 0, nb_a = nb_next, nb_b = 0;
    if (whole > 1) {
      sm_b = sm_at(1);
      if constexpr (NORM) nb_b = nb_at(1, wide);
    }
    uint32_t gq = 0;
    for (; gq + 1 < whole; gq += 2) {
      full_group(gq, sm_a, nb_a, wide);
      sm_a = sm_at(gq + 2);
      if constexpr (NORM) nb_a = nb_at(gq + 2, wide);
      full_group(gq + 1, sm_b, nb_b, wide);
      sm_b = sm_at(gq + 3);
      if constexpr (NORM) nb_b = nb_at(gq + 3, wide);
    }
    if (gq < whole) full_group(gq, sm_a, nb_a, wide);
  };
  if (!NORM || nm.log2n >= 3) full_groups(NzConst<1>{});
  else full_groups(NzConst<0>{});
  if (!GEMV && whole < body) {  // the ragged last group of the tensor
    const uint32_t idx0 = (whole * NZ_LANES + lane) * NZ_GROUP;
    uint32_t ew[8];
    w.group(ew);
    if (idx0 < seg_n) {
      const uint32_t rem = seg_n - idx0 < 8 ? seg_n - idx0 : 8;
      for (uint32_t j = 0; j < rem; ++j) {
        const uint32_t bit = (idx0 + j) * (S + 1);
        const uint32_t rp = ((uint32_t)pk[bit >> 3] >> (7u - S - (bit & 7u))) & ((2u << S) - 1u);
        uint32_t sym = 0;
#pragma unroll
        for (int q = 0; q < 8; ++q) sym = (uint32_t)q == j ? (ew[q] >> 24) : sym;
        uint32_t h = nz_merge_one<S>(sym, rp);
        if constexpr (NORM) h = nz_norm_mul(h, nm.bytes[(seg_base + idx0 + j) >> nm.log2n]);
        dst[idx0 + j] = (uint16_t)h;
      }
    }
  }
  uint32_t ext[2][8];
#pragma unroll
  for (uint32_t t = 0; t < 2; ++t)
    if (t < tailg) w.group(ext[t]);

  // every lane must be back at the encoder's start state (2^16 | carried bits)
  // and the wave must not have read past its record
  const bool bad = (carry ? (w.x >> 16) != 1u : w.x != NZ_L) || (w.base > w.nwords);
  if (__ballot(bad) != 0 && lane == 0) atomicOr(d_status, 4u);

  if (carry) {
    // the ring is dead now: park the 128 carried bytes at its start
    reinterpret_cast<uint16_t*>(w.ring32)[lane] = (uint16_t)(w.x & 0xFFFFu);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const uint8_t* tailp = reinterpret_cast<const uint8_t*>(w.ring32);
#pragma unroll
    for (uint32_t t = 0; t < 2; ++t) {
      if (t < tailg) {
        const uint32_t idx0 = ((body + t) * NZ_LANES + lane) * NZ_GROUP;
        const uint32_t b = idx0 / 8 * (S + 1);
        const uint64_t sm = b >= keep ? nz_load_sm<S>(tailp + (b - keep)) : nz_load_sm<S>(pk + b);
        uint4 mv = nz_merge_group<S>(sm, ext[t]);
        if constexpr (NORM) mv = nz_scale8<true>(mv, nz_norm_load8(nm, seg_base + idx0), nm.log2n >= 3);
        if constexpr (GEMV) walk.add(mv, walk.load(walk.col), lane);
        else *reinterpret_cast<uint4*>(dst + idx0) = mv;
      }
    }
  }
  if constexpr (GEMV)
    if (walk.pending) walk.flush(lane);
}

template <int S, bool NORM, bool STREAM>
__global__ __launch_bounds__(64 * NZ_MAX_SEGS_PER_CHUNK) void nz_decode_kernel(
    const uint8_t* __restrict__ comp, uint64_t comp_bytes, const uint8_t* __restrict__ packed,
    uint16_t* __restrict__ out, NzGeom g, uint32_t* __restrict__ d_status, const NzNorm nm) {
  nz_decode_chunk<S, 0, NORM, STREAM>(comp, comp_bytes, packed, out, g, d_status, blockIdx.x, NzGemv{}, nm);
}

// Several tensors in one launch: the grid is the concatenation of their
// chunks, `chunk_end` the running total.  The items ride in the kernel
// argument block, so a launch needs no device-side table.
#define NZ_BATCH_MAX 16
struct NzBatchItem {
  const uint8_t* comp;
  uint64_t comp_bytes;
  const uint8_t* packed;
  uint16_t* out;       // dense output (decode) ...
  long long* acc;      // ... or the row accumulators, output and bias (matrix-vector product)
  uint16_t* y;
  const uint16_t* bias;
  const uint8_t* norm; // group bytes of a normalized tensor
  NzGeom g;
  uint32_t chunk_end;
  uint32_t reserved;
};
struct NzBatch {
  uint32_t count;
  uint32_t in_features;  // matrix-vector product only
  const uint16_t* x;     // matrix-vector product only
  uint32_t log2n;        // normalized tensors only
  uint32_t x_rows;       // matrix-vector product only: activation rows (1..8)
  NzBatchItem item[NZ_BATCH_MAX];
};

template <int S, bool NORM, bool STREAM>
__global__ __launch_bounds__(64 * NZ_MAX_SEGS_PER_CHUNK) void nz_decode_batch_kernel(
    const NzBatch b, uint32_t* __restrict__ d_status) {
  uint32_t t = 0, first = 0;
  while (t + 1 < b.count && blockIdx.x >= b.item[t].chunk_end) {
    first = b.item[t].chunk_end;
    ++t;
  }
  const NzBatchItem& it = b.item[t];
  nz_decode_chunk<S, 0, NORM, STREAM>(it.comp, it.comp_bytes, it.packed, it.out, it.g, d_status,
                                          blockIdx.x - first, NzGemv{}, NzNorm{it.norm, b.log2n});
}

// The same walk over several matrices that multiply one activation row, or up
// to MR of them (each decoded weight is then used MR times before it is dropped).
template <int S, bool NORM, int MR>
__global__ __launch_bounds__(64 * NZ_MAX_SEGS_PER_CHUNK) void nz_decode_gemv_kernel(
    const NzBatch b, uint32_t* __restrict__ d_status) {
  uint32_t t = 0, first = 0;
  while (t + 1 < b.count && blockIdx.x >= b.item[t].chunk_end) {
    first = b.item[t].chunk_end;
    ++t;
  }
  const NzBatchItem& it = b.item[t];
  const NzGemv gv{b.x, it.acc, it.y, it.bias, b.in_features, b.x_rows};
  nz_decode_chunk<S, MR, NORM, false>(it.comp, it.comp_bytes, it.packed, nullptr, it.g, d_status,
                                        blockIdx.x - first, gv, NzNorm{it.norm, b.log2n});
}

// ----------------------------------------------------------------------------
// row gather (embedding lookup): decode only the chunks that hold the rows asked
// for.  Workgroup (i, k) decodes the k-th chunk touched by row indices[i] into
// slot i * cpr + k of `scratch` (a slot is one chunk of bf16 values); the copy
// kernel then lifts the row out of its slots.  An index outside the table sets
// status bit 8 and yields a row of zeros.
// ----------------------------------------------------------------------------
template <int S, bool NORM>
__global__ __launch_bounds__(64 * NZ_MAX_SEGS_PER_CHUNK) void nz_decode_rows_kernel(
    const uint8_t* __restrict__ comp, uint64_t comp_bytes, const uint8_t* __restrict__ packed,
    uint16_t* __restrict__ scratch, NzGeom g, uint32_t* __restrict__ d_status, const NzNorm nm,
    const long long* __restrict__ indices, uint32_t row_len, uint32_t cpr) {
  const uint32_t i = blockIdx.x / cpr, k = blockIdx.x - i * cpr;
  const long long idx = indices[i];
  if (idx < 0 || (uint64_t)idx >= g.n / row_len) {
    if (threadIdx.x == 0 && k == 0) atomicOr(d_status, 8u);
    return;
  }
  const uint64_t first = (uint64_t)idx * row_len, last = first + row_len - 1;
  const uint64_t c = first / g.chunk_syms + k;
  if (c > last / g.chunk_syms) return;
  // the chunk function writes element e of the tensor to out[e]: shift `out` so
  // that the chunk's first element lands at the start of this workgroup's slot
  uint16_t* out = scratch + ((int64_t)blockIdx.x - (int64_t)c) * (int64_t)g.chunk_syms;
  // (the slots are read back by the copy kernel right away: ordinary stores)
  nz_decode_chunk<S, 0, NORM, false>(comp, comp_bytes, packed, out, g, d_status, c, NzGemv{}, nm);
}

#ifndef NZ_TEMPLATES_ONLY
// `bx` workgroups per row, rows along the same grid dimension (no limit of
// 65535 rows); `i` counts from the start of the slice the scratch holds.
__global__ __launch_bounds__(256) void nz_copy_rows_kernel(const uint16_t* __restrict__ scratch,
                                                           const long long* __restrict__ indices,
                                                           uint64_t rows, uint32_t row_len,
                                                           uint32_t chunk_syms, uint32_t cpr, uint32_t bx,
                                                           uint16_t* __restrict__ out) {
  const uint32_t i = blockIdx.x / bx, part = blockIdx.x - i * bx;
  const long long idx = indices[i];
  const bool ok = idx >= 0 && (uint64_t)idx < rows;
  const uint64_t first = ok ? (uint64_t)idx * row_len : 0;
  const uint64_t c0 = first / chunk_syms;
  for (uint32_t e = part * 256 + threadIdx.x; e < row_len; e += bx * 256) {
    const uint64_t ge = first + e;
    const uint64_t c = ge / chunk_syms;
    const uint16_t v = ok ? scratch[((uint64_t)i * cpr + (c - c0)) * chunk_syms + (ge - c * chunk_syms)] : 0;
    out[(uint64_t)i * row_len + e] = v;
  }
}
#endif  // NZ_TEMPLATES_ONLY
