/*
 * CPU oracle for the NeuZip bf16 codec path.  TEST INFRASTRUCTURE ONLY
 * (see nz_oracle.h for what is pinned and what is "parity unpinned").
 *
 * Plain C, no dependencies beyond libc + pthreads.
 */
#include "nz_oracle.h"

#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* split / merge: reference cuda/kernels.cuh, bf16 instantiation             */
/*   f_bits = 7, e_bits = 8, value_t = uint16 (cuda/high_level.cu:149-153)   */
/* ------------------------------------------------------------------------- */

size_t nzo_packed_bytes(uint64_t n, int s) {
  /* cuda/high_level.cu:81-83: (size * (f_bits_save + 1) + 7) / 8 */
  return (size_t)((n * (uint64_t)(s + 1) + 7) / 8);
}

static int popc8(unsigned v) {
  int c = 0;
  while (v) {
    c += v & 1;
    v >>= 1;
  }
  return c;
}

void nzo_split_bf16(const uint16_t* data, uint64_t n, int s, uint8_t* exponents,
                    uint8_t* fractions) {
  const int f_bits = 7, e_bits = 8;
  memset(fractions, 0, nzo_packed_bytes(n, s));
  for (uint64_t idx = 0; idx < n; ++idx) {
    uint16_t value = data[idx];
    /* kernels.cuh:122 */
    uint8_t sign = (value >> (f_bits + e_bits)) & 0x1;
    /* kernels.cuh:123 */
    uint8_t repr = (uint8_t)(value & ((1 << f_bits) - 1));
    /* kernels.cuh:126-127 */
    uint8_t carry = (f_bits > s) ? ((repr >> (f_bits - s - 1)) & 1) : 0;
    /* kernels.cuh:129 */
    uint8_t exponent = (value >> f_bits) & ((1 << e_bits) - 1);
    /* kernels.cuh:132 */
    repr = repr >> (f_bits - s);
    /* kernels.cuh:134 */
    uint8_t overflow = (uint8_t)((popc8(repr) == s) & carry);
    /* kernels.cuh:137 */
    repr = (uint8_t)((sign << s) | (((1 << s) - 1) & (repr + carry)));
    /* kernels.cuh:86-89,140-149: the warp reduce sums the pre-shifted fields
       of the elements that share an output byte; fields do not overlap, so
       the sum is an OR.  byte = idx*(s+1)/8, shift = 7 - s - (idx*(s+1) & 7). */
    uint64_t bit = idx * (uint64_t)(s + 1);
    uint32_t shift = 7 - s - (uint32_t)(bit & 7);
    fractions[bit >> 3] |= (uint8_t)(repr << shift);
    /* kernels.cuh:153-155: uint8 store wraps 255+1 -> 0 */
    exponents[idx] = (uint8_t)(exponent + overflow);
  }
}

static inline uint16_t merge_bits(uint8_t exponent, uint8_t fbyte, uint64_t idx, int s) {
  const int f_bits = 7;
  uint32_t shift = 7 - s - (uint32_t)((idx * (uint64_t)(s + 1)) & 7);
  /* kernels.cuh:197 */
  uint16_t e = (uint16_t)(exponent << f_bits);
  /* kernels.cuh:200 */
  uint16_t repr = (uint16_t)(fbyte >> shift);
  /* kernels.cuh:202-203 */
  uint16_t fraction = (uint16_t)((repr & ((1 << s) - 1)) << (f_bits - s));
  /* kernels.cuh:204 */
  uint16_t sign = (repr >> s) & 0x1;
  /* kernels.cuh:206 and :213-216 for every non-NaN value: multiplying by
     +-1.0f and converting back only sets the sign bit. */
  return (uint16_t)((sign << 15) | e | fraction);
}

void nzo_merge_bf16(const uint8_t* exponents, const uint8_t* fractions, uint64_t n, int s,
                    uint16_t* data) {
  for (uint64_t idx = 0; idx < n; ++idx) {
    uint64_t bit = idx * (uint64_t)(s + 1);
    data[idx] = merge_bits(exponents[idx], fractions[bit >> 3], idx, s);
  }
}

static inline float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

void nzo_merge_bf16_float(const uint8_t* exponents, const uint8_t* fractions, uint64_t n, int s,
                          uint16_t* data) {
  for (uint64_t idx = 0; idx < n; ++idx) {
    uint64_t bit = idx * (uint64_t)(s + 1);
    uint16_t assembled = merge_bits(exponents[idx], fractions[bit >> 3], idx, s);
    uint16_t sign = assembled >> 15;
    uint16_t value = assembled & 0x7FFF; /* exponent | fraction, kernels.cuh:206 */
    /* kernels.cuh:213-216: 1.0f * float(bf16(value)) * (sign ? -1 : 1) -> bf16 */
    float f = 1.0f * bits_to_float((uint32_t)value << 16) * (sign ? -1.0f : 1.0f);
    uint32_t u = float_to_bits(f);
    uint16_t out;
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
      out = 0x7FC0; /* c10 host round_to_nearest_even NaN rule */
    } else {
      uint32_t bias = 0x7FFFu + ((u >> 16) & 1u);
      out = (uint16_t)((u + bias) >> 16);
    }
    data[idx] = out;
  }
}

/* ---- block normalizers: kernels.cuh:94-118 (split side), :208-216 (merge side) ----
 *
 * Group j holds the elements [j*norm_size, (j+1)*norm_size) of the flat tensor.
 *   split: absmax = max |float(x)| over the group (:97-100; elements past the end
 *          count as 0, :92); fraction = the 23 mantissa bits of absmax (:104,
 *          _float_to_fraction :36-38); every element is divided by the float
 *          1.fraction (:108-112, _fraction_to_base_float :31-34) and cast back
 *          to bf16, round to nearest even; the group stores fraction >> 15
 *          (:116).  A bf16 absmax has 7 mantissa bits, so the stored byte loses
 *          nothing: byte = mantissa << 1.
 *   merge: out = bf16( 1.(byte << 15) * float(value) * +-1 )  (:208-216).
 * The reference reduces with cub::BlockReduce<float, norm_size> inside a block of
 * 1024 threads, which is only well defined for norm_size == 1024; for the other
 * sizes this restates the intended group-wise maximum.  NaN inputs: the order of
 * a float max with NaN operands is unspecified there -> PARITY UNPINNED; here the
 * maximum is taken over the 15-bit magnitude patterns.
 */
static inline uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = float_to_bits(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

size_t nzo_norm_count(uint64_t n, uint32_t norm_size) {
  return norm_size ? (size_t)((n + norm_size - 1) / norm_size) : 0;
}

void nzo_block_normalize(const uint16_t* data, uint64_t n, uint32_t norm_size, uint8_t* norm_bytes,
                         uint16_t* scaled) {
  for (uint64_t g0 = 0; g0 < n; g0 += norm_size) {
    uint64_t g1 = g0 + norm_size < n ? g0 + norm_size : n;
    uint32_t amax = 0; /* bit pattern of |x|: ordered like the value for non-NaN */
    for (uint64_t i = g0; i < g1; ++i) {
      uint32_t a = data[i] & 0x7FFFu;
      if (a > amax) amax = a;
    }
    uint32_t fraction = float_to_bits(bits_to_float(amax << 16)) & 0x7FFFFFu; /* :36-38 */
    float base = bits_to_float((0x7Fu << 23) | fraction);                      /* :31-34 */
    norm_bytes[g0 / norm_size] = (uint8_t)(fraction >> (23 - 8));              /* :116 */
    for (uint64_t i = g0; i < g1; ++i) {
      float x = bits_to_float((uint32_t)data[i] << 16);
      scaled[i] = f32_to_bf16_rne(x / base); /* :111-112 */
    }
  }
}

void nzo_block_denormalize(const uint16_t* scaled, uint64_t n, uint32_t norm_size,
                           const uint8_t* norm_bytes, uint16_t* data) {
  for (uint64_t i = 0; i < n; ++i) {
    float base = bits_to_float((0x7Fu << 23) | ((uint32_t)norm_bytes[i / norm_size] << (23 - 8)));
    uint16_t v = scaled[i];
    float mag = bits_to_float((uint32_t)(v & 0x7FFFu) << 16);
    data[i] = f32_to_bf16_rne(base * mag * ((v >> 15) ? -1.0f : 1.0f)); /* :213-216 */
  }
}

uint16_t nzo_recon_closed_form(uint16_t v, int s) {
  /* Independent statement of merge(split(v)): round-half-up of the 15-bit
     magnitude to a multiple of 2^(7-s), wrapping modulo 2^15. */
  if (s >= 7) return v;
  uint16_t a = v & 0x7FFF;
  uint16_t r = (uint16_t)(((a + (1u << (6 - s))) & 0x7FFFu) & ~((1u << (7 - s)) - 1u));
  return (uint16_t)((v & 0x8000) | r);
}

/* ------------------------------------------------------------------------- */
/* frequency tables                                                          */
/* ------------------------------------------------------------------------- */

/* Quantise a histogram to 12-bit frequencies that sum to exactly 4096.
   Every live symbol first receives one slot, the remaining 4096-K slots are
   shared out by floor(cnt * (4096-K) / n), and the slots still missing go to
   the most frequent symbol (lowest index on ties).  A chunk with one live
   symbol gets 4095 + a single slot for its neighbour (sym ^ 1) so that every
   frequency fits 12 bits.  Returns the most frequent symbol (the pad symbol). */
int nzo_normalize_freqs(const uint32_t cnt[256], uint64_t n, uint16_t freq[256]) {
  uint32_t k = 0;
  for (int i = 0; i < 256; ++i) k += cnt[i] > 0;
  memset(freq, 0, 256 * sizeof(uint16_t));
  if (k == 0 || n == 0) { /* empty chunk: any valid table */
    freq[0] = 4095;
    freq[1] = 1;
    return 0;
  }
  uint32_t sum = 0, best = 0;
  int imax = -1;
  for (int i = 0; i < 256; ++i) {
    if (!cnt[i]) continue;
    uint32_t f = 1 + (uint32_t)(((uint64_t)cnt[i] * (NZO_M - k)) / n);
    freq[i] = (uint16_t)f;
    sum += f;
    if (imax < 0 || cnt[i] > best) {
      best = cnt[i];
      imax = i;
    }
  }
  freq[imax] = (uint16_t)(freq[imax] + (NZO_M - sum));
  if (k == 1) {
    freq[imax] = NZO_M - 1;
    freq[imax ^ 1] = 1;
  }
  return imax;
}

static void put12(uint8_t* p, uint32_t i, uint32_t v) {
  uint32_t bit = 12 * i;
  uint8_t* q = p + (bit >> 3);
  if (bit & 4) {
    q[0] = (uint8_t)((q[0] & 0x0F) | ((v & 0xF) << 4));
    q[1] = (uint8_t)(v >> 4);
  } else {
    q[0] = (uint8_t)(v & 0xFF);
    q[1] = (uint8_t)((q[1] & 0xF0) | (v >> 8));
  }
}
static uint32_t get12(const uint8_t* p, uint32_t i) {
  uint32_t bit = 12 * i;
  const uint8_t* q = p + (bit >> 3);
  uint32_t w = (uint32_t)q[0] | ((uint32_t)q[1] << 8);
  return (w >> (bit & 4)) & 0xFFF;
}

/* Table record:
     byte 0      R = number of maximal runs of live symbols if 1..15,
                 0 = bitmap form (more than 15 runs)
     runs form   R x (start u8, len-1 u8)
     bitmap form 32 bytes, bit (s & 7) of byte (s >> 3) set when s is live
     then        K 12-bit frequencies (field i at bit 12*i, little endian),
                 one per live symbol in ascending symbol order
     zero padding to a multiple of 4 bytes. */
size_t nzo_table_serialize(const uint16_t freq[256], uint8_t* out) {
  uint32_t runs = 0, k = 0;
  for (int i = 0; i < 256; ++i) {
    if (freq[i]) {
      ++k;
      if (i == 0 || !freq[i - 1]) ++runs;
    }
  }
  size_t head;
  memset(out, 0, 420);
  if (runs >= 1 && runs <= NZO_MAX_RUNS) {
    out[0] = (uint8_t)runs;
    uint32_t r = 0;
    for (int i = 0; i < 256; ++i) {
      if (freq[i] && (i == 0 || !freq[i - 1])) {
        int j = i;
        while (j < 256 && freq[j]) ++j;
        out[1 + 2 * r] = (uint8_t)i;
        out[2 + 2 * r] = (uint8_t)(j - i - 1);
        ++r;
      }
    }
    head = 1 + 2 * (size_t)runs;
  } else {
    out[0] = NZO_MODE_BITMAP;
    for (int i = 0; i < 256; ++i)
      if (freq[i]) out[1 + (i >> 3)] |= (uint8_t)(1u << (i & 7));
    head = 33;
  }
  uint32_t j = 0;
  for (int i = 0; i < 256; ++i)
    if (freq[i]) put12(out + head, j++, freq[i]);
  size_t bytes = head + (12 * (size_t)k + 7) / 8;
  return (bytes + 3) & ~(size_t)3;
}

int nzo_table_parse(const uint8_t* in, size_t avail, uint16_t freq[256], size_t* used) {
  memset(freq, 0, 256 * sizeof(uint16_t));
  if (avail < 4) return NZO_ERR_CORRUPT;
  uint8_t live[256];
  memset(live, 0, sizeof live);
  size_t head;
  uint32_t k = 0;
  uint32_t r = in[0];
  if (r >= 1 && r <= NZO_MAX_RUNS) {
    head = 1 + 2 * (size_t)r;
    if (avail < head) return NZO_ERR_CORRUPT;
    int prev_end = -1;
    for (uint32_t i = 0; i < r; ++i) {
      int start = in[1 + 2 * i], len = in[2 + 2 * i] + 1;
      if (start <= prev_end || start + len > 256) return NZO_ERR_CORRUPT;
      for (int j = start; j < start + len; ++j) live[j] = 1;
      prev_end = start + len; /* next run must leave a gap */
      k += (uint32_t)len;
    }
  } else if (r == NZO_MODE_BITMAP) {
    head = 33;
    if (avail < head) return NZO_ERR_CORRUPT;
    for (int i = 0; i < 256; ++i) {
      live[i] = (in[1 + (i >> 3)] >> (i & 7)) & 1;
      k += live[i];
    }
  } else {
    return NZO_ERR_CORRUPT;
  }
  size_t bytes = head + (12 * (size_t)k + 7) / 8;
  bytes = (bytes + 3) & ~(size_t)3;
  if (avail < bytes) return NZO_ERR_CORRUPT;
  uint32_t j = 0, sum = 0;
  for (int i = 0; i < 256; ++i) {
    if (!live[i]) continue;
    uint32_t f = get12(in + head, j++);
    if (f == 0) return NZO_ERR_CORRUPT;
    freq[i] = (uint16_t)f;
    sum += f;
  }
  if (sum != NZO_M) return NZO_ERR_CORRUPT;
  *used = bytes;
  return NZO_OK;
}

/* ------------------------------------------------------------------------- */
/* container geometry                                                        */
/* ------------------------------------------------------------------------- */

typedef struct {
  uint64_t n;
  uint32_t chunk_syms, lane_syms, seg_syms, spc;
  uint64_t n_chunks, n_segs;
  size_t dir_off, rec_off;
} geom_t;

int nzo_check_geometry(uint32_t chunk_syms, uint32_t lane_syms) {
  if (lane_syms < 16 || lane_syms % NZO_GROUP) return NZO_ERR_ARG;
  if (lane_syms > (1u << 16)) return NZO_ERR_ARG;
  uint64_t seg = (uint64_t)lane_syms * NZO_LANES;
  if (chunk_syms == 0 || chunk_syms % NZO_GROUP_SYMS || chunk_syms > (1u << 24)) return NZO_ERR_ARG;
  /* a chunk is cut into spc segments of 64 * lane_syms symbols, the last one
     holding what remains (at least 1024 symbols, so that it can carry 128 bytes) */
  uint64_t spc = (chunk_syms + seg - 1) / seg;
  if (spc < 1 || spc > 8) return NZO_ERR_ARG;
  if (chunk_syms - (spc - 1) * seg < 1024) return NZO_ERR_ARG;
  return NZO_OK;
}

static int make_geom(geom_t* g, uint64_t n, uint32_t chunk_syms, uint32_t lane_syms) {
  if (nzo_check_geometry(chunk_syms, lane_syms)) return NZO_ERR_ARG;
  g->n = n;
  g->chunk_syms = chunk_syms;
  g->lane_syms = lane_syms;
  g->seg_syms = lane_syms * NZO_LANES;
  g->spc = (chunk_syms + g->seg_syms - 1) / g->seg_syms;
  g->n_chunks = (n + chunk_syms - 1) / chunk_syms;
  /* segment c * spc + k is the k-th segment of chunk c; a ragged last chunk has fewer */
  g->n_segs = (n / chunk_syms) * g->spc + ((n % chunk_syms) + g->seg_syms - 1) / g->seg_syms;
  if (g->n_segs >= 0xFFFFFFFEull) return NZO_ERR_ARG;
  g->dir_off = NZO_HEADER_BYTES;
  g->rec_off = (NZO_HEADER_BYTES + 4 * (size_t)(g->n_segs + 1) + 15) & ~(size_t)15;
  return NZO_OK;
}

/* symbols segment k of a chunk holds when the tensor does not end inside it */
static uint32_t seg_nominal(const geom_t* g, uint32_t k) {
  return k + 1 < g->spc ? g->seg_syms : g->chunk_syms - (g->spc - 1) * g->seg_syms;
}

/* worst-case bytes of one segment record holding seg_n symbols */
static size_t seg_rec_cap(const geom_t* g) {
  /* table (<= 420) + states (<= 272) + words (at most one per symbol) ; RAW: 4 + seg_syms + 128 */
  return 420 + 272 + 2 * (size_t)g->seg_syms + 8;
}

size_t nzo_exp_bound(uint64_t n, uint32_t chunk_syms, uint32_t lane_syms) {
  geom_t g;
  if (make_geom(&g, n, chunk_syms, lane_syms)) return 0;
  /* a chunk is never stored larger than its RAW form: 4 per chunk, and per
     segment pad4(seg_n) symbols + 128 carried bytes */
  return g.rec_off + (size_t)n + (4 + 2 * NZO_LANES) * (size_t)g.n_segs + 4 * (size_t)g.n_chunks +
         NZO_TAIL_PAD;
}

static void put32(uint8_t* p, uint32_t v) {
  p[0] = (uint8_t)v;
  p[1] = (uint8_t)(v >> 8);
  p[2] = (uint8_t)(v >> 16);
  p[3] = (uint8_t)(v >> 24);
}
static uint32_t get32(const uint8_t* p) {
  return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}
static void put16(uint8_t* p, uint32_t v) {
  p[0] = (uint8_t)v;
  p[1] = (uint8_t)(v >> 8);
}
static uint32_t get16(const uint8_t* p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8); }

/* ------------------------------------------------------------------------- */
/* segment encode / decode: 64 lanes, lane l owns symbols (g*64+l)*8 + j     */
/* ------------------------------------------------------------------------- */

/* Final encoder states, variable length: 64 two-bit length codes (lane l at
   bits 2l, 2l+1 of a 16-byte little-endian block; code c means the state is
   stored in 5 + c nibbles), then the states as a little-endian nibble stream in
   lane order, zero padded to a multiple of 4 bytes.  A state is >= 2^16, so it
   needs 20..32 bits; storing only the nibbles in use saves about 4 bits per
   lane over a flat 32. */
static size_t pack_states(const uint32_t x[NZO_LANES], uint8_t* out) {
  uint8_t nib[NZO_LANES * 8 + 8];
  size_t t = 0;
  memset(out, 0, 16);
  for (int l = 0; l < NZO_LANES; ++l) {
    uint32_t c = 0;
    while (c < 3 && (x[l] >> (4 * (5 + c))) != 0) ++c;
    out[(2 * l) >> 3] |= (uint8_t)(c << ((2 * l) & 7));
    for (uint32_t k = 0; k < 5 + c; ++k) nib[t++] = (x[l] >> (4 * k)) & 0xF;
  }
  size_t bytes = ((t + 1) / 2 + 3) & ~(size_t)3;
  memset(out + 16, 0, bytes);
  for (size_t k = 0; k < t; ++k) out[16 + (k >> 1)] |= (uint8_t)(nib[k] << (4 * (k & 1)));
  return 16 + bytes;
}

static int unpack_states(const uint8_t* rec, size_t avail, uint32_t x[NZO_LANES], size_t* used) {
  if (avail < 16) return NZO_ERR_CORRUPT;
  size_t t = 0;
  uint32_t n[NZO_LANES];
  for (int l = 0; l < NZO_LANES; ++l) {
    n[l] = 5 + ((rec[(2 * l) >> 3] >> ((2 * l) & 7)) & 3);
    t += n[l];
  }
  size_t bytes = ((t + 1) / 2 + 3) & ~(size_t)3;
  if (avail < 16 + bytes) return NZO_ERR_CORRUPT;
  size_t k = 0;
  for (int l = 0; l < NZO_LANES; ++l) {
    uint32_t v = 0;
    for (uint32_t q = 0; q < n[l]; ++q, ++k)
      v |= (uint32_t)((rec[16 + (k >> 1)] >> (4 * (k & 1))) & 0xF) << (4 * q);
    x[l] = v;
  }
  *used = 16 + bytes;
  return NZO_OK;
}

/* Encode one segment.  Words are produced back to front into words[cap_words]
   so that the decoder reads them front to back.  Returns the number of words,
   or -1 when more than cap_words would be needed (segment stored RAW). */
static int64_t encode_segment(const uint8_t* syms, uint32_t seg_n, int pad_sym,
                              const uint16_t* freq, const uint16_t* cum, const uint16_t* seeds,
                              uint16_t* words, uint32_t cap_words, uint32_t states[NZO_LANES]) {
  uint32_t x[NZO_LANES];
  /* the encoder's start state carries 16 payload bits per lane (see header) */
  for (int l = 0; l < NZO_LANES; ++l) x[l] = NZO_L | (seeds ? seeds[l] : 0u);
  uint32_t ngroups = (seg_n + NZO_GROUP_SYMS - 1) / NZO_GROUP_SYMS;
  uint32_t pos = cap_words;
  for (uint32_t g = ngroups; g-- > 0;) {
    for (int j = NZO_GROUP - 1; j >= 0; --j) {
      uint8_t sym[NZO_LANES];
      uint8_t need[NZO_LANES];
      uint32_t cnt = 0;
      for (int l = 0; l < NZO_LANES; ++l) {
        uint32_t idx = (g * NZO_LANES + (uint32_t)l) * NZO_GROUP + (uint32_t)j;
        sym[l] = idx < seg_n ? syms[idx] : (uint8_t)pad_sym;
        need[l] = x[l] >= ((uint32_t)freq[sym[l]] << 20);
        cnt += need[l];
      }
      if (cnt > pos) return -1;
      pos -= cnt;
      uint32_t p = 0;
      for (int l = 0; l < NZO_LANES; ++l) {
        if (need[l]) {
          words[pos + p++] = (uint16_t)(x[l] & 0xFFFF);
          x[l] >>= 16;
        }
        uint32_t f = freq[sym[l]];
        x[l] = ((x[l] / f) << NZO_PROB_BITS) + (x[l] % f) + cum[sym[l]];
      }
    }
  }
  for (int l = 0; l < NZO_LANES; ++l) states[l] = x[l];
  /* move to the front of the buffer */
  uint32_t count = cap_words - pos;
  memmove(words, words + pos, (size_t)count * 2);
  return count;
}

static int decode_segment(const uint8_t* rec, size_t rec_bytes, uint32_t seg_n,
                          const uint32_t* lut, uint8_t* out, uint16_t* seeds) {
  uint32_t x[NZO_LANES];
  size_t sbytes;
  if (unpack_states(rec, rec_bytes, x, &sbytes)) return NZO_ERR_CORRUPT;
  for (int l = 0; l < NZO_LANES; ++l)
    if (x[l] < NZO_L) return NZO_ERR_CORRUPT;
  const uint8_t* w = rec + sbytes;
  size_t nwords = (rec_bytes - sbytes) / 2, base = 0;
  uint32_t ngroups = (seg_n + NZO_GROUP_SYMS - 1) / NZO_GROUP_SYMS;
  for (uint32_t g = 0; g < ngroups; ++g) {
    for (int j = 0; j < NZO_GROUP; ++j) {
      for (int l = 0; l < NZO_LANES; ++l) {
        uint32_t e = lut[x[l] & (NZO_M - 1)];
        x[l] = (e >> 20) * (x[l] >> NZO_PROB_BITS) + ((e >> 8) & 0xFFF);
        uint32_t idx = (g * NZO_LANES + (uint32_t)l) * NZO_GROUP + (uint32_t)j;
        if (idx < seg_n) out[idx] = (uint8_t)(e & 0xFF);
        if (x[l] < NZO_L) {
          uint32_t word = base < nwords ? get16(w + 2 * base) : 0;
          ++base;
          x[l] = (x[l] << 16) | word;
        }
      }
    }
  }
  if (base > nwords) return NZO_ERR_CORRUPT;
  for (int l = 0; l < NZO_LANES; ++l) {
    /* back at the encoder's start state: 2^16 | payload (payload 0 when nothing is carried) */
    if ((x[l] >> 16) != 1u) return NZO_ERR_CORRUPT;
    if (seeds) seeds[l] = (uint16_t)(x[l] & 0xFFFFu);
    else if (x[l] != NZO_L) return NZO_ERR_CORRUPT;
  }
  return NZO_OK;
}

/* ------------------------------------------------------------------------- */
/* chunk level                                                               */
/* ------------------------------------------------------------------------- */

typedef struct {
  const geom_t* g;
  const uint8_t* syms;
  const uint16_t* seeds; /* 64 per full segment, or NULL */
  uint8_t* scratch;      /* n_segs * seg_rec_cap */
  uint32_t* seg_bytes;   /* n_segs */
  uint64_t c0, c1;       /* chunk range */
} enc_job_t;

static void encode_chunk(const geom_t* g, const uint8_t* syms, const uint16_t* seeds, uint64_t c,
                         uint8_t* scratch, uint32_t* seg_bytes) {
  uint64_t base = c * g->chunk_syms;
  uint64_t cn64 = g->n - base < g->chunk_syms ? g->n - base : g->chunk_syms;
  uint32_t cn = (uint32_t)cn64;
  const uint8_t* cs = syms + base;
  uint32_t cnt[256];
  memset(cnt, 0, sizeof cnt);
  for (uint32_t i = 0; i < cn; ++i) cnt[cs[i]]++;
  uint16_t freq[256], cum[256];
  int pad = nzo_normalize_freqs(cnt, cn, freq);
  uint32_t acc = 0;
  for (int i = 0; i < 256; ++i) {
    cum[i] = (uint16_t)acc;
    acc += freq[i];
  }
  uint8_t table[420];
  size_t tbytes = nzo_table_serialize(freq, table);
  uint32_t nseg = (cn + g->seg_syms - 1) / g->seg_syms;
  uint64_t seg0 = c * g->spc;
  size_t cap = seg_rec_cap(g);
  size_t rans_total = tbytes, raw_total = 4;
  int overflow = 0;
  for (uint32_t k = 0; k < nseg; ++k) {
    uint32_t sn = cn - k * g->seg_syms < g->seg_syms ? cn - k * g->seg_syms : g->seg_syms;
    uint8_t* rec = scratch + (seg0 + k) * cap;
    size_t off = 0;
    if (k == 0) {
      memcpy(rec, table, tbytes);
      off = tbytes;
    }
    uint32_t states[NZO_LANES];
    uint16_t* words = (uint16_t*)malloc(2 * (size_t)g->seg_syms + 8);
    /* only full segments carry payload in their start states */
    const uint16_t* sd = (seeds && sn == seg_nominal(g, k)) ? seeds + (seg0 + k) * NZO_LANES : NULL;
    /* one word per symbol is the most a segment can emit: no overflow */
    int64_t nw = encode_segment(cs + (size_t)k * g->seg_syms, sn, pad, freq, cum, sd, words,
                                g->seg_syms, states);
    if (nw < 0) {
      overflow = 1;
      nw = 0;
    }
    off += pack_states(states, rec + off);
    for (int64_t i = 0; i < nw; ++i) put16(rec + off + 2 * i, words[i]);
    off += 2 * (size_t)nw;
    if (nw & 1) {
      put16(rec + off, 0);
      off += 2;
    }
    free(words);
    seg_bytes[seg0 + k] = (uint32_t)off;
    rans_total += off - (k == 0 ? tbytes : 0);
    raw_total += (((size_t)sn + 3) & ~(size_t)3) + (sn == seg_nominal(g, k) ? 2 * NZO_LANES : 0);
  }
  if (overflow || rans_total >= raw_total) {
    for (uint32_t k = 0; k < nseg; ++k) {
      uint32_t sn = cn - k * g->seg_syms < g->seg_syms ? cn - k * g->seg_syms : g->seg_syms;
      uint8_t* rec = scratch + (seg0 + k) * cap;
      size_t off = 0;
      if (k == 0) {
        rec[0] = NZO_MODE_RAW;
        rec[1] = rec[2] = rec[3] = 0;
        off = 4;
      }
      memcpy(rec + off, cs + (size_t)k * g->seg_syms, sn);
      size_t padded = ((size_t)sn + 3) & ~(size_t)3;
      memset(rec + off + sn, 0, padded - sn);
      off += padded;
      if (sn == seg_nominal(g, k)) { /* a raw full segment still has to hold its 64 x 16 carried bits */
        for (int l = 0; l < NZO_LANES; ++l)
          put16(rec + off + 2 * l, seeds ? seeds[(seg0 + k) * NZO_LANES + l] : 0u);
        off += 2 * NZO_LANES;
      }
      seg_bytes[seg0 + k] = (uint32_t)off;
    }
  }
}

static void* enc_worker(void* arg) {
  enc_job_t* j = (enc_job_t*)arg;
  for (uint64_t c = j->c0; c < j->c1; ++c)
    encode_chunk(j->g, j->syms, j->seeds, c, j->scratch, j->seg_bytes);
  return NULL;
}

static void write_header(uint8_t* out, const geom_t* g, uint64_t total) {
  memset(out, 0, NZO_HEADER_BYTES);
  put32(out + 0, NZO_MAGIC);
  put32(out + 4, NZO_VERSION);
  put32(out + 8, (uint32_t)(g->n & 0xFFFFFFFFu));
  put32(out + 12, (uint32_t)(g->n >> 32));
  put32(out + 16, g->chunk_syms);
  put32(out + 20, g->lane_syms);
  put32(out + 24, (uint32_t)g->n_chunks);
  put32(out + 28, (uint32_t)g->n_segs);
  put32(out + 32, (uint32_t)g->dir_off);
  put32(out + 36, (uint32_t)g->rec_off);
  put32(out + 40, (uint32_t)(total & 0xFFFFFFFFu));
  put32(out + 44, (uint32_t)(total >> 32));
}

int64_t nzo_exp_encode(const uint8_t* syms, uint64_t n, uint32_t chunk_syms, uint32_t lane_syms,
                       const uint16_t* seeds, uint8_t* out, size_t cap, int threads) {
  geom_t g;
  if (make_geom(&g, n, chunk_syms, lane_syms)) return NZO_ERR_ARG;
  if (cap < g.rec_off) return NZO_ERR_CAP;
  size_t rcap = seg_rec_cap(&g);
  uint8_t* scratch = (uint8_t*)malloc((size_t)g.n_segs * rcap + 1);
  uint32_t* seg_bytes = (uint32_t*)calloc((size_t)g.n_segs + 1, 4);
  if (!scratch || !seg_bytes) {
    free(scratch);
    free(seg_bytes);
    return NZO_ERR_CAP;
  }
  if (threads < 1) threads = 1;
  if ((uint64_t)threads > g.n_chunks) threads = g.n_chunks ? (int)g.n_chunks : 1;
  pthread_t* tid = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
  enc_job_t* jobs = (enc_job_t*)malloc(sizeof(enc_job_t) * (size_t)threads);
  for (int t = 0; t < threads; ++t) {
    jobs[t].g = &g;
    jobs[t].syms = syms;
    jobs[t].seeds = seeds;
    jobs[t].scratch = scratch;
    jobs[t].seg_bytes = seg_bytes;
    jobs[t].c0 = g.n_chunks * (uint64_t)t / (uint64_t)threads;
    jobs[t].c1 = g.n_chunks * (uint64_t)(t + 1) / (uint64_t)threads;
    if (threads == 1)
      enc_worker(&jobs[t]);
    else
      pthread_create(&tid[t], NULL, enc_worker, &jobs[t]);
  }
  if (threads > 1)
    for (int t = 0; t < threads; ++t) pthread_join(tid[t], NULL);
  free(tid);
  free(jobs);

  int64_t ret;
  uint64_t units = 0;
  memset(out + NZO_HEADER_BYTES, 0, g.rec_off - NZO_HEADER_BYTES);
  for (uint64_t k = 0; k < g.n_segs; ++k) {
    put32(out + g.dir_off + 4 * k, (uint32_t)units);
    size_t at = g.rec_off + 4 * (size_t)units;
    if (at + seg_bytes[k] > cap) {
      ret = NZO_ERR_CAP;
      goto done;
    }
    memcpy(out + at, scratch + k * rcap, seg_bytes[k]);
    units += seg_bytes[k] / 4;
    if (units > 0xFFFFFFFFull) {
      ret = NZO_ERR_ARG;
      goto done;
    }
  }
  put32(out + g.dir_off + 4 * g.n_segs, (uint32_t)units);
  {
    /* 16 zero bytes close the container so that 16-byte loads of the last
       words never leave it */
    uint64_t total = g.rec_off + 4 * units + NZO_TAIL_PAD;
    if (total > cap) {
      ret = NZO_ERR_CAP;
      goto done;
    }
    memset(out + g.rec_off + 4 * units, 0, NZO_TAIL_PAD);
    write_header(out, &g, total);
    ret = (int64_t)total;
  }
done:
  free(scratch);
  free(seg_bytes);
  return ret;
}

static void build_lut(const uint16_t freq[256], uint32_t* lut) {
  uint32_t c = 0;
  for (int s = 0; s < 256; ++s) {
    uint32_t f = freq[s];
    for (uint32_t i = 0; i < f; ++i) lut[c + i] = (f << 20) | (i << 8) | (uint32_t)s;
    c += f;
  }
}

typedef struct {
  const geom_t* g;
  const uint8_t* comp;
  size_t comp_bytes;
  uint8_t* out;
  uint16_t* seeds; /* 64 per full segment, or NULL */
  uint64_t c0, c1;
  int status;
} dec_job_t;

static int decode_chunk(const geom_t* g, const uint8_t* comp, size_t comp_bytes, uint64_t c,
                        uint8_t* out, uint16_t* seeds) {
  uint64_t base = c * g->chunk_syms;
  uint32_t cn = (uint32_t)(g->n - base < g->chunk_syms ? g->n - base : g->chunk_syms);
  uint32_t nseg = (cn + g->seg_syms - 1) / g->seg_syms;
  uint64_t seg0 = c * g->spc;
  const uint8_t* dir = comp + g->dir_off;
  uint32_t lut[NZO_M];
  int raw = 0;
  for (uint32_t k = 0; k < nseg; ++k) {
    uint64_t o0 = get32(dir + 4 * (seg0 + k)), o1 = get32(dir + 4 * (seg0 + k + 1));
    if (o1 < o0 || g->rec_off + 4 * o1 > comp_bytes) return NZO_ERR_CORRUPT;
    const uint8_t* rec = comp + g->rec_off + 4 * o0;
    size_t rbytes = 4 * (size_t)(o1 - o0);
    uint32_t sn = cn - k * g->seg_syms < g->seg_syms ? cn - k * g->seg_syms : g->seg_syms;
    uint8_t* dst = out + base + (size_t)k * g->seg_syms;
    if (k == 0) {
      if (rbytes < 4) return NZO_ERR_CORRUPT;
      if (rec[0] == NZO_MODE_RAW) {
        raw = 1;
        rec += 4;
        rbytes -= 4;
      } else {
        uint16_t freq[256];
        size_t used;
        if (nzo_table_parse(rec, rbytes, freq, &used)) return NZO_ERR_CORRUPT;
        build_lut(freq, lut);
        rec += used;
        rbytes -= used;
      }
    }
    uint16_t tmp[NZO_LANES];
    uint16_t* sd = sn == seg_nominal(g, k) ? (seeds ? seeds + (seg0 + k) * NZO_LANES : tmp) : NULL;
    if (raw) {
      size_t padded = ((size_t)sn + 3) & ~(size_t)3;
      if (rbytes < padded + (sd ? 2 * NZO_LANES : 0)) return NZO_ERR_CORRUPT;
      memcpy(dst, rec, sn);
      if (sd)
        for (int l = 0; l < NZO_LANES; ++l) sd[l] = (uint16_t)get16(rec + padded + 2 * l);
    } else {
      int r = decode_segment(rec, rbytes, sn, lut, dst, sd);
      if (r) return r;
    }
  }
  return NZO_OK;
}

static void* dec_worker(void* arg) {
  dec_job_t* j = (dec_job_t*)arg;
  j->status = NZO_OK;
  for (uint64_t c = j->c0; c < j->c1; ++c) {
    int r = decode_chunk(j->g, j->comp, j->comp_bytes, c, j->out, j->seeds);
    if (r) {
      j->status = r;
      break;
    }
  }
  return NULL;
}

int nzo_exp_decode(const uint8_t* comp, size_t comp_bytes, uint64_t n, uint8_t* syms_out,
                   uint16_t* seeds_out, int threads) {
  if (comp_bytes < NZO_HEADER_BYTES) return NZO_ERR_CORRUPT;
  if (get32(comp) != NZO_MAGIC || get32(comp + 4) != NZO_VERSION) return NZO_ERR_CORRUPT;
  uint64_t hn = (uint64_t)get32(comp + 8) | ((uint64_t)get32(comp + 12) << 32);
  if (hn != n) return NZO_ERR_CORRUPT;
  geom_t g;
  if (make_geom(&g, n, get32(comp + 16), get32(comp + 20))) return NZO_ERR_CORRUPT;
  if (get32(comp + 24) != (uint32_t)g.n_chunks || get32(comp + 28) != (uint32_t)g.n_segs ||
      get32(comp + 32) != g.dir_off || get32(comp + 36) != g.rec_off)
    return NZO_ERR_CORRUPT;
  uint64_t total = (uint64_t)get32(comp + 40) | ((uint64_t)get32(comp + 44) << 32);
  if (total > comp_bytes || total < g.rec_off) return NZO_ERR_CORRUPT;
  if (g.rec_off + 4 * (uint64_t)get32(comp + g.dir_off + 4 * g.n_segs) + NZO_TAIL_PAD != total)
    return NZO_ERR_CORRUPT;
  if (threads < 1) threads = 1;
  if ((uint64_t)threads > g.n_chunks) threads = g.n_chunks ? (int)g.n_chunks : 1;
  pthread_t* tid = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
  dec_job_t* jobs = (dec_job_t*)malloc(sizeof(dec_job_t) * (size_t)threads);
  int status = NZO_OK;
  for (int t = 0; t < threads; ++t) {
    jobs[t].g = &g;
    jobs[t].comp = comp;
    jobs[t].comp_bytes = (size_t)total - NZO_TAIL_PAD;
    jobs[t].out = syms_out;
    jobs[t].seeds = seeds_out;
    jobs[t].c0 = g.n_chunks * (uint64_t)t / (uint64_t)threads;
    jobs[t].c1 = g.n_chunks * (uint64_t)(t + 1) / (uint64_t)threads;
    if (threads == 1)
      dec_worker(&jobs[t]);
    else
      pthread_create(&tid[t], NULL, dec_worker, &jobs[t]);
  }
  for (int t = 0; t < threads; ++t) {
    if (threads > 1) pthread_join(tid[t], NULL);
    if (jobs[t].status) status = jobs[t].status;
  }
  free(tid);
  free(jobs);
  return status;
}

/* ------------------------------------------------------------------------- */
/* whole tensor: reference _write_to_cache (cuda/high_level.cu:76-130) and   */
/* _decompress_and_merge (:169-206) with the container above in place of     */
/* nvcomp.                                                                   */
/* ------------------------------------------------------------------------- */

typedef struct {
  const uint16_t* data;
  uint16_t* out;
  uint8_t* exps;
  uint8_t* fractions;
  uint64_t i0, i1;
  int s;
} sm_job_t;

static void* split_worker(void* arg) {
  sm_job_t* j = (sm_job_t*)arg;
  /* ranges are multiples of 8 elements, so packed bytes do not straddle jobs */
  uint64_t b0 = j->i0 * (uint64_t)(j->s + 1) / 8;
  nzo_split_bf16(j->data + j->i0, j->i1 - j->i0, j->s, j->exps + j->i0, j->fractions + b0);
  return NULL;
}
static void* merge_worker(void* arg) {
  sm_job_t* j = (sm_job_t*)arg;
  uint64_t b0 = j->i0 * (uint64_t)(j->s + 1) / 8;
  nzo_merge_bf16(j->exps + j->i0, j->fractions + b0, j->i1 - j->i0, j->s, j->out + j->i0);
  return NULL;
}

static void run_sm(void* (*fn)(void*), const uint16_t* data, uint16_t* out, uint8_t* exps,
                   uint8_t* fractions, uint64_t n, int s, int threads) {
  if (threads < 1) threads = 1;
  if (n < 4096) threads = 1;
  pthread_t* tid = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
  sm_job_t* jobs = (sm_job_t*)malloc(sizeof(sm_job_t) * (size_t)threads);
  for (int t = 0; t < threads; ++t) {
    jobs[t].data = data;
    jobs[t].out = out;
    jobs[t].exps = exps;
    jobs[t].fractions = fractions;
    jobs[t].s = s;
    jobs[t].i0 = (n * (uint64_t)t / (uint64_t)threads) & ~(uint64_t)7;
    jobs[t].i1 = t == threads - 1 ? n : ((n * (uint64_t)(t + 1) / (uint64_t)threads) & ~(uint64_t)7);
    if (threads == 1)
      fn(&jobs[t]);
    else
      pthread_create(&tid[t], NULL, fn, &jobs[t]);
  }
  if (threads > 1)
    for (int t = 0; t < threads; ++t) pthread_join(tid[t], NULL);
  free(tid);
  free(jobs);
}

/* Stored layout of the packed sign|mantissa stream: the reference layout
   (byte idx*(s+1)/8, MSB first) with the last 128 bytes of every FULL segment
   taken out; those 64 x 16 bits ride in the start states of the segment's 64
   rANS lanes (lane l carries bytes 2l and 2l+1, little endian).  A segment is
   full when the tensor does not end inside it. */
static uint64_t full_segments(const geom_t* g) {
  uint64_t rem = g->n % g->chunk_syms, fs = rem / g->seg_syms;
  if (fs > g->spc - 1) fs = g->spc - 1;
  return (g->n / g->chunk_syms) * g->spc + fs;
}

size_t nzo_packed_stored_bytes(uint64_t n, int s, uint32_t chunk_syms, uint32_t lane_syms) {
  geom_t g;
  if (make_geom(&g, n, chunk_syms, lane_syms)) return 0;
  return nzo_packed_bytes(n, s) - 2 * NZO_LANES * (size_t)full_segments(&g);
}

/* move the packed bytes between the reference layout (`full`) and the stored
   layout + per-segment carried bytes */
static void carry_layout(const geom_t* g, int s, uint8_t* full, uint8_t* stored, uint16_t* seeds,
                         int to_stored) {
  size_t total = nzo_packed_bytes(g->n, s), src = 0, dst = 0;
  for (uint64_t c = 0; c < g->n_chunks; ++c) {
    uint64_t base = c * g->chunk_syms;
    uint32_t cn = (uint32_t)(g->n - base < g->chunk_syms ? g->n - base : g->chunk_syms);
    uint32_t nseg = (cn + g->seg_syms - 1) / g->seg_syms;
    for (uint32_t k = 0; k < nseg; ++k) {
      uint32_t sn = cn - k * g->seg_syms < g->seg_syms ? cn - k * g->seg_syms : g->seg_syms;
      int is_full = sn == seg_nominal(g, k);
      size_t bytes = is_full ? (size_t)sn * (size_t)(s + 1) / 8 : total - src;
      size_t keep = is_full ? bytes - 2 * NZO_LANES : bytes;
      if (to_stored) memcpy(stored + dst, full + src, keep);
      else memcpy(full + src, stored + dst, keep);
      if (is_full) {
        uint16_t* sd = seeds + (c * g->spc + k) * NZO_LANES;
        for (int l = 0; l < NZO_LANES; ++l) {
          if (to_stored) sd[l] = (uint16_t)get16(full + src + keep + 2 * l);
          else put16(full + src + keep + 2 * l, sd[l]);
        }
      }
      src += bytes;
      dst += keep;
    }
  }
}

int64_t nzo_compress_bf16(const uint16_t* data, uint64_t n, int s, uint32_t chunk_syms,
                          uint32_t lane_syms, uint8_t* fractions, uint8_t* comp, size_t cap,
                          int threads) {
  if (!(s == 7 || s == 3 || s == 1 || s == 0)) return NZO_ERR_ARG;
  geom_t g;
  if (make_geom(&g, n, chunk_syms, lane_syms)) return NZO_ERR_ARG;
  uint8_t* exps = (uint8_t*)malloc((size_t)n + 1);
  uint8_t* full = (uint8_t*)malloc(nzo_packed_bytes(n, s) + 1);
  uint16_t* seeds = (uint16_t*)calloc((size_t)(g.n_segs + 1) * NZO_LANES, 2);
  if (!exps || !full || !seeds) {
    free(exps);
    free(full);
    free(seeds);
    return NZO_ERR_CAP;
  }
  run_sm(split_worker, data, NULL, exps, full, n, s, threads);
  carry_layout(&g, s, full, fractions, seeds, 1);
  int64_t r = nzo_exp_encode(exps, n, chunk_syms, lane_syms, seeds, comp, cap, threads);
  free(exps);
  free(full);
  free(seeds);
  return r;
}

int nzo_decompress_bf16(const uint8_t* comp, size_t comp_bytes, const uint8_t* fractions,
                        uint64_t n, int s, uint16_t* data, int threads) {
  if (!(s == 7 || s == 3 || s == 1 || s == 0)) return NZO_ERR_ARG;
  if (comp_bytes < NZO_HEADER_BYTES) return NZO_ERR_CORRUPT;
  geom_t g;
  if (make_geom(&g, n, get32(comp + 16), get32(comp + 20))) return NZO_ERR_CORRUPT;
  uint8_t* exps = (uint8_t*)malloc((size_t)n + 1);
  uint8_t* full = (uint8_t*)malloc(nzo_packed_bytes(n, s) + 1);
  uint16_t* seeds = (uint16_t*)calloc((size_t)(g.n_segs + 1) * NZO_LANES, 2);
  if (!exps || !full || !seeds) {
    free(exps);
    free(full);
    free(seeds);
    return NZO_ERR_CAP;
  }
  int r = nzo_exp_decode(comp, comp_bytes, n, exps, seeds, threads);
  if (r == NZO_OK) {
    carry_layout(&g, s, full, (uint8_t*)fractions, seeds, 0);
    run_sm(merge_worker, NULL, data, exps, full, n, s, threads);
  }
  free(exps);
  free(full);
  free(seeds);
  return r;
}
