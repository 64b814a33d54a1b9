// Container geometry shared by the host API and the gfx950 kernels.
//
// The exponent stream of one tensor (N bytes, one per bf16 element) is stored
// as
//
//   header (64 B) | directory ((n_segs + 1) x u32) | segment records | 16 zero bytes
//
// * chunk   = `chunk_syms` consecutive exponents that share one 12-bit
//             frequency table (the reference hands nvcomp the same unit:
//             chunk_size = 65536, cuda/neuzip.cu:31).
// * segment = 64 * `lane_syms` consecutive exponents decoded by ONE wavefront:
//             64 interleaved rANS states, lane l owning the 8-symbol groups
//             (g * 64 + l) * 8 + j.  A chunk is cut into spc = 1..8 segments,
//             the last one holding what remains of the chunk (>= 1024
//             symbols); segment c * spc + k is the k-th segment of chunk c.
// * directory entry k = offset of segment k's record in 4-byte units from
//             `rec_off`; entry n_segs = end of the last record.
// * record  = [table, first segment of a chunk only] [final encoder states:
//             64 two-bit length codes (lane l at bits 2l, 2l+1; code c = the
//             state takes 5 + c nibbles) and the states as a little-endian
//             nibble stream in lane order, padded to 4 bytes] [u16
//             renormalisation words, front-to-back in decode order] padded to
//             4 bytes; or, for a chunk whose coded form
//             would not be smaller, [0xFF 0 0 0, first segment only] raw
//             exponent bytes padded to 4 [+ 64 x u16 carried bits if full].
// * carry   = the encoder of a FULL segment starts lane l in state
//             2^16 | c_l instead of 2^16, where c_l are bytes 2l, 2l+1 of the
//             last 128 bytes of the segment's packed sign|mantissa stream.
//             Those 128 bytes are not stored in the packed stream (every full
//             segment stores NZ_CARRY_BYTES fewer); the decoder finds them in
//             the low halves of its final states.  This returns 16 of the
//             ~24 bits that flushing a 32-bit rANS state costs per lane.
#pragma once

#include <stddef.h>
#include <stdint.h>

#ifdef __HIPCC__
#define NZ_HD __host__ __device__
#else
#define NZ_HD
#endif

#define NZ_MAGIC 0x315A4E41u
#define NZ_FORMAT_VERSION 4u
#define NZ_PROB_BITS 12
#define NZ_M (1u << NZ_PROB_BITS)
#define NZ_L (1u << 16)
#define NZ_LANES 64
#define NZ_GROUP 8
#define NZ_GROUP_SYMS 512
#define NZ_HEADER_BYTES 64
#define NZ_MODE_RAW 0xFF
#define NZ_MODE_BITMAP 0x00
#define NZ_MAX_RUNS 15
#define NZ_TABLE_MAX_BYTES 424 /* 1 + 32 + 384 rounded up to a multiple of 8 */
#define NZ_MAX_SEGS_PER_CHUNK 8
#define NZ_CARRY_BYTES 128 /* 64 lanes x 16 bits */
#define NZ_STATE_MAX_BYTES 272 /* 16 bytes of length codes + 64 x 32 bits */
#define NZ_TAIL_PAD 16     /* zero bytes after the last record: 16-byte loads stay inside */

struct NzGeom {
  uint64_t n;
  uint32_t chunk_syms;
  uint32_t lane_syms;
  uint32_t seg_syms;
  uint32_t spc;  // segments per chunk
  uint64_t n_chunks;
  uint64_t n_segs;
  uint64_t dir_off;
  uint64_t rec_off;
};

// Device-side per-chunk record produced by the split/histogram kernel.
struct NzChunkInfo {
  uint32_t tab_len;  // serialized table bytes (multiple of 4)
  uint32_t pad_sym;  // most frequent symbol: stands in for elements past the end
  uint32_t raw;      // 1 when the chunk is stored raw
  uint32_t reserved;
};

static inline int nz_geom_check(uint32_t chunk_syms, uint32_t lane_syms) {
  if (lane_syms < 16 || (lane_syms % NZ_GROUP) != 0 || lane_syms > (1u << 16)) return -1;
  uint64_t seg = (uint64_t)lane_syms * NZ_LANES;
  if (chunk_syms == 0 || (chunk_syms % NZ_GROUP_SYMS) != 0 || chunk_syms > (1u << 24)) return -1;
  uint64_t spc = (chunk_syms + seg - 1) / seg;
  if (spc < 1 || spc > NZ_MAX_SEGS_PER_CHUNK) return -1;
  if (chunk_syms - (spc - 1) * seg < 1024) return -1;  // the last segment must be able to carry 128 bytes
  return 0;
}

static inline int nz_geom_make(NzGeom* g, uint64_t n, uint32_t chunk_syms, uint32_t lane_syms) {
  if (nz_geom_check(chunk_syms, lane_syms)) return -1;
  g->n = n;
  g->chunk_syms = chunk_syms;
  g->lane_syms = lane_syms;
  g->seg_syms = lane_syms * NZ_LANES;
  g->spc = (chunk_syms + g->seg_syms - 1) / g->seg_syms;
  g->n_chunks = (n + chunk_syms - 1) / chunk_syms;
  g->n_segs = (n / chunk_syms) * g->spc + ((n % chunk_syms) + g->seg_syms - 1) / g->seg_syms;
  if (g->n_segs >= 0xFFFFFFFEull) return -1;
  g->dir_off = NZ_HEADER_BYTES;
  g->rec_off = (NZ_HEADER_BYTES + 4 * (g->n_segs + 1) + 15) & ~(uint64_t)15;
  return 0;
}

// Upper bound of the container size: no chunk is ever stored larger than raw.
static inline uint64_t nz_geom_bound(const NzGeom* g) {
  return g->rec_off + g->n + (4 + NZ_CARRY_BYTES) * g->n_segs + 4 * g->n_chunks + NZ_TAIL_PAD;
}

static inline uint64_t nz_packed_bytes_of(uint64_t n, int s) {
  return (n * (uint64_t)(s + 1) + 7) / 8;  // cuda/high_level.cu:81-83
}

// Symbols segment k of a chunk holds when the tensor does not end inside it.
NZ_HD static inline uint32_t nz_seg_nominal(uint32_t chunk_syms, uint32_t seg_syms, uint32_t spc, uint32_t k) {
  return k + 1 < spc ? seg_syms : chunk_syms - (spc - 1) * seg_syms;
}

// Segments the tensor does not end inside ("full": they carry 128 packed bytes).
static inline uint64_t nz_full_segments(const NzGeom* g) {
  uint64_t rem = g->n % g->chunk_syms, fs = rem / g->seg_syms;
  if (fs > g->spc - 1) fs = g->spc - 1;
  return (g->n / g->chunk_syms) * g->spc + fs;
}

// Bytes actually stored for the packed stream: the reference size minus the
// carried bytes of every full segment.
static inline uint64_t nz_packed_stored_bytes_of(const NzGeom* g, int s) {
  return nz_packed_bytes_of(g->n, s) - (uint64_t)NZ_CARRY_BYTES * nz_full_segments(g);
}
