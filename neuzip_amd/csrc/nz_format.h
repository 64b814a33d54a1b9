// Container geometry shared by the host API and the gfx950 kernels.
//
// The exponent stream of one tensor (N bytes, one per bf16 element) is stored
// as
//
//   header (64 B) | directory ((n_segs + 1) x u32) | segment records | 16 zero bytes
//
// * chunk   = `chunk_syms` consecutive exponents that share one 12-bit
//             frequency table and are decoded by one workgroup (the reference
//             hands nvcomp chunk_size = 65536, cuda/neuzip.cu:31).
// * segment = 64 * `lane_syms` consecutive exponents decoded by ONE wavefront:
//             lane l owns the 8-symbol groups (g * 64 + l) * 8 + j and codes
//             them with two table-ANS states (A: even j, B: odd j) into one
//             private bit stream.  A chunk is cut into spc = 1..8 segments,
//             the last one holding what remains of the chunk (>= 1536
//             symbols); segment c * spc + k is the k-th segment of chunk c.
// * directory entry k = offset of segment k's record in 4-byte units from
//             `rec_off`; entry n_segs = end of the last record.
// * record  = [table, first segment of a chunk only] [states: 64 x 24 bits,
//             lane l at bytes 3l .. 3l+2, state A in the low 12 bits]
//             [u32 minlen | w << 24] [64 fields of w bits: len_l - minlen]
//             [the 64 lane streams back to back, bit-granular, little endian]
//             padded to 4 bytes; or, for a chunk whose coded form would not be
//             smaller, [0xFF 0 0 0, first segment only] raw exponent bytes
//             padded to 4 [+ the carried bytes if full].
// * coder   = table ANS with T = 4096 states.  Slot i of [0, T) belongs to the
//             symbol whose cumulative 12-bit frequency range holds i; state X
//             stands on slot (X % 64) * 64 + X / 64; the k-th state of symbol
//             s in ascending order stands for x = f_s + k: the decoder reads
//             n = 12 - floor(log2 x) bits b and moves to (x << n) - T + b.  A
//             lane's stream is read from its end downwards, A's bits above
//             B's for each pair of symbols.
// * carry   = the encoder of a FULL segment starts the two states of lane l
//             from T | 12 payload bits each: bytes 3l .. 3l+2 of the last
//             NZ_CARRY_BYTES bytes of the segment's packed sign|mantissa
//             stream, which are not stored in the packed stream; the decoder
//             finds them in its final states.  So the 24 bits a lane's start
//             states cost in the record are paid back.
#pragma once

#include <stddef.h>
#include <stdint.h>

#ifdef __HIPCC__
#define NZ_HD __host__ __device__
#else
#define NZ_HD
#endif

#define NZ_MAGIC 0x315A4E41u
#define NZ_FORMAT_VERSION 5u
#define NZ_PROB_BITS 12
#define NZ_M (1u << NZ_PROB_BITS)
#define NZ_LANES 64
#define NZ_GROUP 8
#define NZ_GROUP_SYMS 512
#define NZ_HEADER_BYTES 64
#define NZ_MODE_RAW 0xFF
#define NZ_MODE_BITMAP 0x00
#define NZ_MAX_RUNS 15
#define NZ_TABLE_MAX_BYTES 424 /* 1 + 32 + 384 rounded up to a multiple of 8 */
#define NZ_MAX_SEGS_PER_CHUNK 8
#define NZ_CARRY_BYTES 192 /* 64 lanes x 2 states x 12 bits */
#define NZ_STATES_BYTES 192
#define NZ_LENS_MAX_BYTES 196 /* u32 header + 64 fields of up to 24 bits */
#define NZ_BODY_HEAD_MAX (NZ_STATES_BYTES + NZ_LENS_MAX_BYTES)
#define NZ_MAX_LANE_SYMS 512u
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
  if (lane_syms < 24 || (lane_syms % NZ_GROUP) != 0 || lane_syms > NZ_MAX_LANE_SYMS) return -1;
  uint64_t seg = (uint64_t)lane_syms * NZ_LANES;
  if (chunk_syms == 0 || (chunk_syms % NZ_GROUP_SYMS) != 0 || chunk_syms > (1u << 24)) return -1;
  uint64_t spc = (chunk_syms + seg - 1) / seg;
  if (spc < 1 || spc > NZ_MAX_SEGS_PER_CHUNK) return -1;
  if (chunk_syms - (spc - 1) * seg < 8 * NZ_CARRY_BYTES) return -1;  // the last segment must be able to carry 192 bytes
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

// Segments the tensor does not end inside ("full": they carry NZ_CARRY_BYTES packed bytes).
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

// Bytes of the scratch slot of one segment: the record body (states, lengths,
// lane streams of up to 12 bits per symbol with one spare dword each) when it
// is not assembled in LDS, or the raw exponent bytes of a chunk stored raw.
NZ_HD static inline uint32_t nz_slot_lane_dwords(uint32_t lane_syms) { return (lane_syms * NZ_PROB_BITS + 31) / 32 + 2; }
NZ_HD static inline uint64_t nz_slot_bytes(uint32_t lane_syms) {
  return (uint64_t)NZ_BODY_HEAD_MAX + 4ull * NZ_LANES * nz_slot_lane_dwords(lane_syms) + 12;
}
