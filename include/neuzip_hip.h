/*
 * C ABI of libneuzip_hip.so: the MI355X (gfx950) NeuZip bf16 codec.
 *
 * This is the drop-in boundary for the reference's pybind11 extension
 * `neuzip._cuda` (cuda/neuzip.cu:19-38): every entry point below names the
 * reference method it stands in for.  Plain pointers and sizes only; device
 * pointers are HIP device addresses, `stream` is a hipStream_t passed as
 * void* (NULL = the default stream).  All kernels are enqueued on the
 * caller's stream; nothing here creates a private stream (the reference's
 * private `estream`, cuda/high_level.cu:47, is not synchronised with the
 * producer of its input and is not reproduced).
 *
 * Every function returns NZ_OK or a negative NZ_ERR_* code; a message for the
 * last failure on the calling thread is available from nz_last_error().
 *
 * Dense bf16 pointers must be 16-byte aligned.
 */
#ifndef NEUZIP_HIP_H
#define NEUZIP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NZ_OK 0
#define NZ_ERR_ARG -1       /* bad argument / unsupported geometry           */
#define NZ_ERR_DTYPE -2     /* "Unsupported data type", high_level.cu:160    */
#define NZ_ERR_NOT_FOUND -3 /* "Data not found", high_level.cu:225           */
#define NZ_ERR_HIP -4       /* a HIP runtime call failed                     */
#define NZ_ERR_CAPACITY -5  /* output buffer too small                       */
#define NZ_ERR_CORRUPT -6   /* compressed buffer failed validation           */
#define NZ_ERR_ALIGN -7     /* dense pointer not 16-byte aligned             */
#define NZ_ERR_ALGO -8      /* "Unsupported algorithm", high_level.cu:67     */

/* dtype codes (only bf16 is implemented; the reference's fp16/fp32 branches,
   high_level.cu:144-161, truncate the mantissa and are out of scope) */
#define NZ_DTYPE_BF16 0
#define NZ_DTYPE_F16 1
#define NZ_DTYPE_F32 2

/* algorithm codes: cuda/algorithms.cuh:8. Only ANS exists here. */
#define NZ_ALGO_ANS 0

/* The library's own geometry (chunk_size 0): tables shared by 128 Ki elements,
   eight wavefronts of 256 symbols per lane each.  The reference hands nvcomp
   chunks of 64 Ki (cuda/neuzip.cu:31); that size is honoured when asked for,
   cut into four segments of 256 symbols per lane. */
#define NZ_DEFAULT_CHUNK 131072u
#define NZ_DEFAULT_LANE_SYMS 256u
#define NZ_LANE_SYMS_AUTO 0xFFFFFFFFu /* nz_manager_create: choose per tensor */
/* Size budget of a manager's own geometry choices: stored exponent bytes
   (container and all) over the order-0 entropy of the exponents, estimated
   from the geometry for weights of ~2.55 bits per exponent.  The reference's
   nvcomp cannot be measured here; this is the stand-in for "within 1 % of
   nvcomp ANS". */
#define NZ_DEFAULT_SIZE_BUDGET 1.01

typedef struct nz_manager nz_manager;

int nz_abi_version(void);
const char* nz_last_error(void);

/* ---- sizes ------------------------------------------------------------ */

/* Packed sign+mantissa bytes for n elements at `precision` kept mantissa
   bits: (n * (precision + 1) + 7) / 8, cuda/high_level.cu:81-83. */
uint64_t nz_packed_bytes(uint64_t n, int precision);

/* Bytes actually stored for the packed stream: the last 128 bytes of every
   full segment (a chunk is cut into segments of 64 * lane_syms elements, the
   last one shorter) travel inside the entropy coder's start states instead
   (16 bits per rANS lane), so each full segment stores 128 bytes fewer than
   the reference layout. */
uint64_t nz_packed_stored_bytes(uint64_t n, int precision, uint32_t chunk_size, uint32_t lane_syms);

/* Capacity that always holds the entropy-coded exponent container of n
   elements (stands in for nvcomp's max_compressed_buffer_size,
   cuda/high_level.cu:106-108).  0 for an unsupported geometry. */
uint64_t nz_exp_bound_bytes(uint64_t n, uint32_t chunk_size, uint32_t lane_syms);

/* Device scratch needed by nz_encode for n elements. */
uint64_t nz_encode_workspace_bytes(uint64_t n, uint32_t chunk_size, uint32_t lane_syms);

/* Bytes of the block-normalizer array of n elements: one byte per group of
   `normalizer_size` consecutive elements (cuda/high_level.cu:89-93), 0 without
   normalizers.  normalizer_size is 0 or a power of two up to 1024, the sizes
   cuda/neuzip.cu:47-105 instantiates. */
uint64_t nz_norm_bytes(uint64_t n, uint32_t normalizer_size);

/* ---- stateless kernels ------------------------------------------------ */

/* Block normalizers (cuda/kernels.cuh:94-118 and :208-216) are part of the
   three calls below: with normalizer_size > 0 every group of that many elements
   is divided by 1.m before the split (m = the mantissa of the group's largest
   magnitude; the byte m << 1 goes to dev_norm, nz_norm_bytes() bytes, 8-byte
   aligned) and multiplied by it after the merge, both rounded to bf16.  With
   normalizer_size == 0 dev_norm is ignored. */

/* Manager::split, cuda/high_level.cu:265-321: unpacked exponent byte and
   sign|mantissa byte per element, precision forced to 7 (:289).  dev_norm is
   scratch here (the reference drops the bytes, :282-296). */
int nz_split(const void* dev_bf16, uint64_t n, void* dev_exponents, void* dev_fractions,
             uint32_t normalizer_size, void* dev_norm, void* stream);

/* Manager::_write_to_cache, cuda/high_level.cu:76-130: split, then entropy
   code the exponents.  `dev_packed` receives nz_packed_stored_bytes() bytes,
   `dev_comp` (capacity comp_cap >= nz_exp_bound_bytes) the container.
   `dev_total` (device uint64) receives the container size, `dev_status`
   (device uint32, OR-ed into) stays zero when the container is complete: bit 0
   = it did not fit, bit 2 = a workgroup gave up waiting for the record sizes
   of the chunks before its own (see nz_set_lookback_spins; the container is
   then incomplete and the call has to be made again; the workspace is marked,
   and the next call that uses it sets bit 2 once more and takes the mark
   away).  The call may be captured into a HIP graph and replayed: the
   workspace keeps a count of the runs that have used it.  If `host_total` is not
   NULL the call synchronises the stream, returns the size and status on the
   host (the reference's get_compressed_output_size sync, :114-115) and deals
   with bit 2 itself.  With host_total NULL (and in nz_encode_static, and in
   every replay of a captured call) nobody does: the caller has to look at
   *dev_status before the container is used, and encode again when bit 2 is
   set.  dev_bf16 is read until the stream has passed the call: it must stay
   valid and unmodified until then. */
int nz_encode(const void* dev_bf16, uint64_t n, int precision, uint32_t chunk_size,
              uint32_t lane_syms, void* dev_packed, void* dev_comp, uint64_t comp_cap,
              void* dev_workspace, uint64_t workspace_bytes, uint64_t* dev_total,
              uint32_t* dev_status, uint64_t* host_total, uint32_t normalizer_size, void* dev_norm,
              void* stream);

/* nz_encode for callers that cannot allocate or hand over a workspace (code
   under HIP graph capture, tight serving loops, harnesses that forbid
   hipMalloc).  No counterpart in the reference.  Same kernels, arguments and
   results as nz_encode, but the scratch is a fixed array of
   NZ_STATIC_SCRATCH_BYTES inside the library's code object (every GPU the
   library runs on holds its own copy until the process ends), and the call
   never allocates, frees or synchronises: the container size is delivered in
   *dev_total only.  A tensor whose nz_encode_workspace_bytes() exceeds
   NZ_STATIC_SCRATCH_BYTES is refused with NZ_ERR_CAPACITY (at the default
   geometry: more than about 5.5 million elements).  All calls on one GPU share
   that GPU's array: calls that overlap in time on one GPU (two streams, two
   threads) race; order them on one stream or with events.  *dev_status has to
   be checked before the container is used: bit 0 (it did not fit) and bit 2 (a
   workgroup gave up waiting, see nz_set_lookback_spins) both leave it
   incomplete, and this call cannot repair either. */
#define NZ_STATIC_SCRATCH_BYTES (16u << 20)
int nz_encode_static(const void* dev_bf16, uint64_t n, int precision, uint32_t chunk_size,
                     uint32_t lane_syms, void* dev_packed, void* dev_comp, uint64_t comp_cap,
                     uint64_t* dev_total, uint32_t* dev_status, uint32_t normalizer_size, void* dev_norm,
                     void* stream);

/* No counterpart in the reference.  The encode kernel of the calls above (and
   of the manager's writes into existing buffers) places its records itself:
   every workgroup waits until the workgroups of the chunks before its own have
   announced their record sizes.  That the workgroups of a launch start in the
   order of their numbers, so that everything waited for is running or done,
   is what has been observed on this device, not something the hardware
   promises: the eight dies dispatch independently, and two encode launches
   that are resident at once (two managers on two streams) can each hold
   compute units while waiting for a predecessor that has not been given one.
   So the wait is bounded: after `spins` looks at an announcement (about a
   microsecond each; default 2^15, some tens of milliseconds - a launch takes
   ~0.1 ms) a workgroup gives up, and the records are placed by a second kernel
   once the host has seen that (at once in nz_encode with host_total; when the
   entry is used next in a manager): a wait that was cut short costs one
   compaction launch, never a wrong container.  For tests and tuning; 0 makes
   every workgroup give up whose predecessors are not done at its first look. */
void nz_set_lookback_spins(uint32_t spins);

/* Manager::_decompress_and_merge, cuda/high_level.cu:169-206: entropy decode
   and merge in one kernel.  `dev_status` (device uint32, zeroed by the
   caller) is OR-ed with a non-zero value when the container fails validation
   (bit 4: the header does not name n / chunk_size / lane_syms as passed).
   `flags`: with NZ_DECODE_CHECK the call synchronises and returns
   NZ_ERR_CORRUPT in that case.  The dense output is written with ordinary
   stores when it is at most 128 MiB (half of the last-level cache: the GEMM
   that consumes a just-decompressed weight then reads it from the cache) and
   with streaming stores when it is larger (it cannot stay resident, and
   streaming keeps it from churning the cache); NZ_DECODE_STREAM_OUT /
   NZ_DECODE_RESIDENT_OUT force one or the other, for a caller who knows that
   nothing will read the output soon / that its consumer runs next.
   chunk_size / lane_syms must be the ones used to encode. */
#define NZ_DECODE_CHECK 1
#define NZ_DECODE_STREAM_OUT 2
#define NZ_DECODE_RESIDENT_OUT 4
int nz_decode(const void* dev_comp, uint64_t comp_bytes, const void* dev_packed, uint64_t n,
              int precision, uint32_t chunk_size, uint32_t lane_syms, void* dev_bf16_out,
              uint32_t* dev_status, int flags, uint32_t normalizer_size, const void* dev_norm,
              void* stream);

/* ---- handle store: template struct Manager, cuda/high_level.cu:26-322 -- */

/* Manager(algorithm, chunk_size) for the class Manager_f{precision}_n{normalizer_size}
   (cuda/neuzip.cu:19-38, neuzip/binding.py:69-70).  precision in {0,1,3,7};
   normalizer_size 0 or a power of two up to 1024 (block normalizers, see above);
   chunk_size 0 selects the library's own table scope.
   lane_syms > 0 is used as given.  lane_syms 0 leaves the segment length to
   the library, which chooses it per tensor: the shortest segments from
   NZ_DEFAULT_LANE_SYMS up whose estimated stored size is within the manager's
   size budget (nz_manager_set_size_budget).  With the library's own chunk these
   are chunks of eight segments: NZ_DEFAULT_CHUNK / NZ_DEFAULT_LANE_SYMS from
   about six million elements up, 264 to 280 symbols per lane for one to four
   million; a given chunk_size of 64 Ki: 344 symbols per lane, three segments.
   NZ_LANE_SYMS_AUTO may, in addition, shorten the segments of a tensor that is
   too small to fill the device: with the library's own chunk it cuts the
   tensor into one, two or three decode workgroups per compute unit (chunks of
   eight segments of 64..512 symbols per lane, in multiples of 8) when that is
   modelled 10 % faster, and a tensor too small for that into 32 Ki chunks of
   eight 4 Ki segments; with a given chunk_size only the segments are
   shortened.  Shorter segments cost ~43 bytes each, so at the default budget
   of 1.01 none qualifies and small tensors keep their size (serve them with
   the batch calls); a larger budget buys wavefronts with bytes.  Every entry
   records the geometry it was written with (nz_manager_geometry). */
int nz_manager_create(int algorithm, int precision, int normalizer_size, uint32_t chunk_size,
                      uint32_t lane_syms, nz_manager** out);
void nz_manager_destroy(nz_manager* m);

/* No counterpart in the reference (nvcomp's ratio is what it is).  The
   manager's own geometry choices (lane_syms 0 or NZ_LANE_SYMS_AUTO at creation)
   keep the estimated stored size of a tensor's exponents within `ratio` x their
   order-0 entropy.  The estimate, for weights of about 2.55 bits per exponent:
   1.0008 + (134.4 x segments + 78 x chunks + 600) / elements, a short last
   segment or chunk counting as a whole one; a geometry is accepted when the
   estimate plus 0.0003, kept in hand for exponents of lower entropy, is within
   the budget.  A tensor so small that no geometry reaches the budget keeps
   the default one.  Default NZ_DEFAULT_SIZE_BUDGET; valid above 1.002 up to 2.
   Affects the writes that follow. */
int nz_manager_set_size_budget(nz_manager* m, double ratio);
double nz_manager_size_budget(const nz_manager* m);
/* The estimate itself for a tensor of n elements (0 for an invalid geometry),
   and whether the manager's own choices would accept the geometry for it, for
   a caller who chooses geometries by hand (nz_manager_geometry_hint). */
double nz_estimated_size_ratio(uint64_t n, uint32_t chunk_size, uint32_t lane_syms);
int nz_manager_in_budget(const nz_manager* m, uint64_t n, uint32_t chunk_size, uint32_t lane_syms);

/* Manager::write(name, tensor), cuda/high_level.cu:132-162.  Replaces an
   existing entry of the same name (:137-140).  Synchronises the stream once
   to learn the compressed size (as the reference does, :114-115), unless the
   handle already holds a tensor of the same element count (see
   nz_manager_rewrite_stats): such a write goes into the entry's buffers and
   returns while the encode kernel is still reading dev_data.  Since a caller
   cannot tell the two cases apart beforehand: dev_data must stay valid and
   unmodified until `stream` has passed the write (free or overwrite it in
   stream order, or after an event / synchronisation; memory from a
   stream-ordered allocator that belongs to another stream has to be told, as
   torch's record_stream does).
   Streams and graphs: writes, products and row gathers of one manager share
   its scratch memory; a call that arrives on another stream than the one
   before it is ordered behind that one on the device (an event, no host
   wait).  A call that may allocate or wait on the host - every write, a read
   or product of an entry whose in-place rewrite has not been looked at yet, a
   product that needs larger accumulators, a row gather - is refused with
   NZ_ERR_ARG while its stream is being captured into a graph, before it
   touches anything (the capture stays valid); reads and products of settled
   entries are captured and replay.  Calls on one manager from several host
   threads are serialised by the manager. */
int nz_manager_write(nz_manager* m, const char* name, const void* dev_data, uint64_t n,
                     int dtype, void* stream);

/* Up to 16 writes together: the tensors ride in the kernel arguments, so split +
   coding of all of them is one launch (one per segment-length class in use),
   their container sizes come back with ONE host synchronisation, then one
   launch fills the exact-size buffers (an optimizer step that re-compresses
   the weights of a block pays one sync instead of one per weight,
   cuda/high_level.cu:114-115 per call).  Same semantics per entry as
   nz_manager_write; a name may appear only once. */
int nz_manager_write_batch(nz_manager* m, const char* const* names, const void* const* dev_data,
                           const uint64_t* ns, uint32_t count, int dtype, void* stream);

/* A write (single or batch) whose handles all hold a tensor of the same element
   count already - the re-compress after an optimizer step,
   neuzip/__init__.py:25-35 - encodes straight into the buffers those entries
   have: no allocation, no free and no wait for the container size, which
   comes back through pinned memory and is looked at when the entry is used
   next (an entry whose container outgrew its buffer, which has ~1.5 % of
   headroom, is then given a larger one and re-compacted from scratch memory
   that is kept until then).  Counters for tests and tuning: batches written in
   place so far, entries that outgrew their buffer, entries whose records were
   placed a second time (see nz_set_lookback_spins).  Settles what is pending. */
int nz_manager_rewrite_stats(nz_manager* m, uint64_t* in_place_batches, uint64_t* outgrown_entries,
                             uint64_t* placed_again);

/* Manager::read(name), cuda/high_level.cu:223-250, into caller-owned memory of
   at least `cap_elems` elements.  Asynchronous on `stream` (the reference
   blocks the host here, :203; callers that need that call hipStreamSynchronize). */
int nz_manager_read(nz_manager* m, const char* name, void* dev_out, uint64_t cap_elems,
                    void* stream);

/* Several Manager::read calls (cuda/high_level.cu:223-250) served by ONE kernel
   launch: entry names[i] is decompressed into dev_outs[i] (capacity
   cap_elems[i] elements).  The reference decompresses tensor by tensor; a
   transformer block's weights are each too small to fill the GPU, together they
   do.  Nothing is decoded when an argument is rejected.  Asynchronous on
   `stream`; allocates nothing. */
int nz_manager_read_batch(nz_manager* m, const char* const* names, void* const* dev_outs,
                          const uint64_t* cap_elems, uint32_t count, void* stream);

/* Manager::linear / linear_without_bias (cuda/high_level.cu:252-263) for ONE
   activation row: y_i = W_i x (+ bias_i) for up to 16 stored matrices W_i =
   names[i] that share the input x, with the weights decoded on the fly and never
   written to memory (the reference decompresses W, then calls matmul).  Each
   stored tensor is read as a row-major matrix with rows of `in_features`
   elements (a multiple of 512).  dev_x: in_features bf16, 16-byte aligned;
   dev_y[i]: rows_i bf16; dev_bias: null, or per matrix null / rows_i bf16.
   Sums are formed in fp32 per wavefront and row; a row that several
   wavefronts share is summed across them in 24.40 fixed point, so the result
   does not depend on scheduling (such a row comes out as NaN when one of its
   partial sums is NaN, infinite or beyond 2^18 in magnitude, and is resolved
   to 2^-40); the wavefront that completes a row rounds and stores it, so the
   whole product is one kernel launch.
   Calls of one manager must be ordered on one stream (they share the
   accumulators, which are allocated on first use and grown when needed; no
   other call allocates).  Asynchronous on `stream`. */
int nz_manager_gemv_batch(nz_manager* m, const char* const* names, uint32_t count, const void* dev_x,
                          uint32_t in_features, const void* const* dev_bias, void* const* dev_y,
                          void* stream);

/* The same for up to NZ_GEMV_MAX_ROWS activation rows (a small batch, or the
   tokens of a speculative step): dev_x holds x_rows rows of in_features values,
   dev_y[i] receives x_rows rows of one value per row of matrix i; every weight
   is decoded once and multiplied with all rows before it is dropped, so the
   call costs little more than the one-row call (Manager::linear for 2-D
   inputs, cuda/high_level.cu:252-263, decodes the weight into memory and runs
   a GEMM over it).  Each output row is, bit for bit, what the one-row call
   gives for that activation row.  Not built for managers with normalizers. */
#define NZ_GEMV_MAX_ROWS 8u
int nz_manager_gemv_rows_batch(nz_manager* m, const char* const* names, uint32_t count,
                               const void* dev_x, uint32_t x_rows, uint32_t in_features,
                               const void* const* dev_bias, void* const* dev_y, void* stream);

/* Embedding lookup on a stored table (neuzip/nn/embedding.py:30-39 decompresses
   the WHOLE table for every forward): row dev_indices[i] (int64) of the table
   `name`, read as rows of row_len elements, goes to dev_out[i * row_len ...];
   only the chunks that hold the requested rows are decoded.  An index outside
   the table gives a row of zeros and makes the next nz_manager_check fail.
   Every (row, chunk) pair is decoded on its own, so a call that asks for about
   as many rows as the table has chunks is better served by nz_manager_read
   (neuzip_amd.Manager.gather_rows makes that choice).  Uses the manager's write
   scratch, at most a quarter GiB of it: larger requests are served in slices
   (calls must be ordered on one stream with the writes).  Asynchronous on
   `stream`. */
int nz_manager_gather_rows(nz_manager* m, const char* name, const void* dev_indices, uint64_t count,
                           uint32_t row_len, void* dev_out, void* stream);

/* Geometry an entry was written with (it travels in the container's header):
   elements per frequency table and symbols per rANS lane and segment. */
int nz_manager_geometry(nz_manager* m, const char* name, uint32_t* chunk_size, uint32_t* lane_syms);

/* No counterpart in the reference (its chunk size is one constructor argument,
   neuzip/binding.py:56-62).  The next writes under `name` use this geometry
   instead of the manager's own choice; (0, 0) takes the hint back.  For tensors
   that are always decoded together by one launch (nz_manager_gemv_batch,
   nz_manager_read_batch): the launch is fastest when the chunks of all of them
   together are a whole number of workgroups per compute unit, which no choice
   per tensor can know (neuzip_amd.FusedGemv.trace uses it).  The write under
   `name` must be serialised with this call by the caller. */
int nz_manager_geometry_hint(nz_manager* m, const char* name, uint32_t chunk_size, uint32_t lane_syms);

/* meta_cache lookup, cuda/high_level.cu:42-43,228-230. */
int nz_manager_meta(nz_manager* m, const char* name, uint64_t* numel, int* dtype);

/* Manager::size(name), cuda/high_level.cu:208-221: bytes held for the entry
   (entropy-coded exponents + packed sign/mantissa + normalizer bytes of a
   manager with normalizer_size > 0); 0 if unknown. */
uint64_t nz_manager_size(nz_manager* m, const char* name);

/* The same figure by the reference's formula, term by term: a manager without
   normalizers also counts the ceil(numel / 1024)-byte buffer the reference
   allocates and never uses (cuda/high_level.cu:89-93, summed at :208-221). */
uint64_t nz_manager_size_reference(nz_manager* m, const char* name);

/* Bytes of the exponent container alone / of the packed stream alone. */
uint64_t nz_manager_exp_bytes(nz_manager* m, const char* name);
uint64_t nz_manager_packed_bytes(nz_manager* m, const char* name);
uint64_t nz_manager_norm_bytes(nz_manager* m, const char* name); /* normalizer bytes, counted in size */

/* Raw device pointers of an entry (valid until it is rewritten or erased). */
int nz_manager_buffers(nz_manager* m, const char* name, const void** dev_comp,
                       uint64_t* comp_bytes, const void** dev_packed, uint64_t* packed_bytes);

/* Copy an entry's streams (container, packed, normalizer bytes) to host memory
   (sizes from nz_manager_exp_bytes / _packed_bytes / _norm_bytes) and back.  The reference keeps compressed tensors
   only inside the process (cuda/high_level.cu:35-43; neuzip/nn/module.py:13
   leaves 0-size parameters in a state_dict), so a converted model cannot be
   checkpointed there; these two calls are what a save/load needs.  The
   container names its own element count and geometry; import checks header,
   directory and sizes against the manager (precision, normalizer_size) and stores
   nothing when they disagree.  Both calls block until the copies are done. */
int nz_manager_export(nz_manager* m, const char* name, void* host_comp, uint64_t comp_cap,
                      void* host_packed, uint64_t packed_cap, void* host_norm, uint64_t norm_cap,
                      void* stream);
int nz_manager_import(nz_manager* m, const char* name, const void* host_comp, uint64_t comp_bytes,
                      const void* host_packed, uint64_t packed_bytes, const void* host_norm,
                      uint64_t norm_bytes, void* stream);

/* Release the manager's scratch (the workspace of the largest write so far, the
   accumulators of the matrix-vector product); it is allocated again on demand.
   The reference allocates its scratch per call (cuda/high_level.cu:81-108).
   Waits for the device. */
int nz_manager_trim(nz_manager* m);

/* compress_cache.erase(name), cuda/high_level.cu:137-140. */
int nz_manager_erase(nz_manager* m, const char* name);

/* Synchronise `stream` and report NZ_ERR_CORRUPT if any read since the last
   check saw a container that failed validation. */
int nz_manager_check(nz_manager* m, void* stream);

#ifdef __cplusplus
}
#endif
#endif
