/*
 * CPU oracle for the NeuZip bf16 codec path.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing in the shipped package may link, import or execute this file: it is
 * the checker that the HIP kernels are compared against (tests, the smoke
 * check and the cpu_baseline leg of the benchmark).
 *
 * Two groups of functions:
 *
 *  1. nzo_split_bf16 / nzo_merge_bf16 restate, line by line, the integer
 *     semantics of the reference kernels
 *        cuda/kernels.cuh:62-156  (kernel_aligned_split, non-normalized bf16)
 *        cuda/kernels.cuh:167-217 (kernel_aligned_merge, non-normalized bf16)
 *     Pinned by: an independent closed form (nzo_recon_closed_form, and a
 *     numpy version of it in the tests) checked on all 65 536 bf16 patterns
 *     for every precision, plus the invariants listed in the tests.
 *     NaN results: the reference multiplies through fp32 and converts back,
 *     which canonicalises NaN payloads in a way that depends on the device
 *     conversion routine -> the exact NaN bit pattern is PARITY UNPINNED.
 *
 *     nzo_block_normalize / nzo_block_denormalize restate the block-normalizer
 *     path (kernels.cuh:94-118, 208-216).  Pinned by an exact rational-arithmetic
 *     model of "divide, round to nearest even" over all mantissa pairs and by
 *     the invariants in the tests; NaN inputs and the reference's behaviour for
 *     group sizes other than 1024 are PARITY UNPINNED (see the source).
 *
 *  2. nzo_exp_* is the chunked, 64-way lane-interleaved rANS container that
 *     replaces the closed-source nvcomp ANS call sites
 *        cuda/high_level.cu:103-124 (compress) and :184-192 (decompress).
 *     The nvcomp bitstream is opaque, so the byte format here is this
 *     project's own; PARITY UNPINNED for the compressed bytes and exact
 *     compressed size.  What is pinned: lossless identity on arbitrary
 *     bytes, the Shannon bound on the size, and textbook rANS state
 *     invariants (checked in the tests).
 */
#ifndef NZ_ORACLE_H
#define NZ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- format constants (shared with the HIP implementation by value) ---- */
#define NZO_MAGIC 0x315A4E41u /* "ANZ1" little endian */
#define NZO_VERSION 4u
#define NZO_PROB_BITS 12
#define NZO_M (1u << NZO_PROB_BITS)
#define NZO_L (1u << 16)
#define NZO_LANES 64
#define NZO_GROUP 8                        /* consecutive symbols per lane per group */
#define NZO_GROUP_SYMS (NZO_LANES * NZO_GROUP) /* 512 */
#define NZO_HEADER_BYTES 64
#define NZO_MODE_RAW 0xFF
#define NZO_MODE_BITMAP 0x00
#define NZO_MAX_RUNS 15
#define NZO_TAIL_PAD 16

/* ---- split / merge ---- */
size_t nzo_packed_bytes(uint64_t n, int s);
size_t nzo_packed_stored_bytes(uint64_t n, int s, uint32_t chunk_syms, uint32_t lane_syms);
void nzo_split_bf16(const uint16_t* data, uint64_t n, int s, uint8_t* exponents, uint8_t* fractions);
void nzo_merge_bf16(const uint8_t* exponents, const uint8_t* fractions, uint64_t n, int s, uint16_t* data);
/* literal float path of kernels.cuh:208-216 (NaN canonicalised to 0x7FC0, host c10 rule) */
void nzo_merge_bf16_float(const uint8_t* exponents, const uint8_t* fractions, uint64_t n, int s,
                          uint16_t* data);
uint16_t nzo_recon_closed_form(uint16_t v, int s);
/* block normalizers (kernels.cuh:94-118, 208-216): one byte per group of norm_size elements */
size_t nzo_norm_count(uint64_t n, uint32_t norm_size);
void nzo_block_normalize(const uint16_t* data, uint64_t n, uint32_t norm_size, uint8_t* norm_bytes,
                         uint16_t* scaled);
void nzo_block_denormalize(const uint16_t* scaled, uint64_t n, uint32_t norm_size,
                           const uint8_t* norm_bytes, uint16_t* data);

/* ---- frequency tables ---- */
int nzo_normalize_freqs(const uint32_t cnt[256], uint64_t n, uint16_t freq[256]);
size_t nzo_table_serialize(const uint16_t freq[256], uint8_t* out);
int nzo_table_parse(const uint8_t* in, size_t avail, uint16_t freq[256], size_t* used);

/* ---- exponent container ---- */
int nzo_check_geometry(uint32_t chunk_syms, uint32_t lane_syms);
size_t nzo_exp_bound(uint64_t n, uint32_t chunk_syms, uint32_t lane_syms);
/* seeds: 64 x u16 per segment (segment c*spc + k at seeds + 64*(c*spc + k); only
   full segments use theirs), the payload carried in the rANS start states;
   NULL = all zero / ignored. */
int64_t nzo_exp_encode(const uint8_t* syms, uint64_t n, uint32_t chunk_syms, uint32_t lane_syms,
                       const uint16_t* seeds, uint8_t* out, size_t cap, int threads);
int nzo_exp_decode(const uint8_t* comp, size_t comp_bytes, uint64_t n, uint8_t* syms_out,
                   uint16_t* seeds_out, int threads);

/* ---- whole tensor (split + encode / decode + merge) ---- */
int64_t nzo_compress_bf16(const uint16_t* data, uint64_t n, int s, uint32_t chunk_syms,
                          uint32_t lane_syms, uint8_t* fractions, uint8_t* comp, size_t cap,
                          int threads);
int nzo_decompress_bf16(const uint8_t* comp, size_t comp_bytes, const uint8_t* fractions,
                        uint64_t n, int s, uint16_t* data, int threads);

/* error codes */
#define NZO_OK 0
#define NZO_ERR_ARG -1
#define NZO_ERR_CAP -2
#define NZO_ERR_CORRUPT -3

#ifdef __cplusplus
}
#endif
#endif
