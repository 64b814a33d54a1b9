// Host side of libneuzip_hip.so: the C ABI declared in include/neuzip_hip.h.
//
// Stands in for the reference's `template struct Manager`
// (cuda/high_level.cu:26-322) and its pybind11 surface (cuda/neuzip.cu:19-38).
// No torch types, no private streams: every kernel goes to the caller's stream.
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>

#include "../../include/neuzip_hip.h"
#include "nz_launch.h"

namespace {

thread_local std::string g_err;

int fail(int code, const std::string& msg) {
  g_err = msg;
  return code;
}

#define NZ_HIP(call)                                                                  \
  do {                                                                                \
    hipError_t e_ = (call);                                                           \
    if (e_ != hipSuccess)                                                             \
      return fail(NZ_ERR_HIP, std::string(#call) + ": " + hipGetErrorString(e_));     \
  } while (0)

inline uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

bool precision_ok(int p) { return p == 7 || p == 3 || p == 1 || p == 0; }

// group sizes the reference instantiates (cuda/neuzip.cu:47-105): 0 = off, else a power of two up to 1024
bool normalizer_ok(uint32_t ns) { return ns == 0 || (ns <= 1024 && (ns & (ns - 1)) == 0); }
uint32_t log2_of(uint32_t v) {
  uint32_t l = 0;
  while ((1u << l) < v) ++l;
  return l;
}
uint64_t norm_bytes_of(uint64_t n, uint32_t ns) { return ns ? (n + ns - 1) / ns : 0; }

// Device scratch of one encode call.
struct EncLayout {
  uint64_t exps, tab_ser, info, carry, slots, states, seg_words, seg_sbytes, seg_units, chunk_units, pub, placed, lb_state, bytes;
};

// segments short enough for the kernel that keeps the exponents in registers
bool enc_in_registers(const NzGeom& g) { return g.lane_syms <= NZ_ENC_MAX_LANE_SYMS; }

EncLayout enc_layout(const NzGeom& g) {
  EncLayout L;
  uint64_t o = 0;
  auto take = [&](uint64_t b) {
    uint64_t at = o;
    o = align_up(o + b, 256);
    return at;
  };
  L.exps = take(enc_in_registers(g) ? 0 : g.n + 16);  // only long segments park their exponents in memory
  L.tab_ser = take(g.n_chunks * NZ_TABLE_MAX_BYTES);
  L.info = take(g.n_chunks * sizeof(NzChunkInfo));
  L.carry = take(g.n_segs * NZ_CARRY_BYTES);
  L.slots = take(g.n_segs * 2 * (uint64_t)g.seg_syms + 16);  // one 2-byte word per symbol: the worst case
  L.states = take(g.n_segs * NZ_STATE_MAX_BYTES);
  L.seg_words = take(g.n_segs * 4);
  L.seg_sbytes = take(g.n_segs * 4);
  L.seg_units = take((g.n_segs + 1) * 4);
  L.chunk_units = take((g.n_chunks + 1) * 4);
  L.pub = take(g.n_chunks * 32);  // size and running-total announcements of the chunks (records placed by the encode kernel)
  L.placed = take(g.n_segs);      // per segment: its record is in the container only
  L.lb_state = take(8);           // run count and abort mark of the announcements
  L.bytes = o;
  return L;
}

// group bytes of a tensor that is about to be split (nothing to do without normalizers)
int launch_absmax(const void* in, uint64_t n, uint32_t ns, uint8_t* norm, hipStream_t st) {
  if (!ns || !n) return NZ_OK;
  hipLaunchKernelGGL(nz_absmax_kernel, dim3((uint32_t)((n + 2047) / 2048)), dim3(256), 0, st,
                     (const uint16_t*)in, n, log2_of(ns), norm);
  NZ_HIP(hipGetLastError());
  return NZ_OK;
}

// A number no earlier call of this process has used and nothing in memory is
// likely to show: it marks the size announcements of one encode call.
uint64_t next_nonce() {
  static std::atomic<uint64_t> ctr{(uint64_t)std::chrono::steady_clock::now().time_since_epoch().count() *
                                   0x9E3779B97F4A7C15ull};
  uint64_t z = ctr.fetch_add(0x9E3779B97F4A7C15ull) + 0x9E3779B97F4A7C15ull;  // splitmix64
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// How often a chunk of a direct encode looks for an announcement it waits for
// (about a microsecond per look) before it gives up: some tens of milliseconds,
// as a wait that is given up costs no more than one compaction kernel.
std::atomic<uint32_t> g_lookback_spins{1u << 15};

// One tensor of an encode call, as the kernels see it.  `comp`/`comp_cap`: where
// the container goes (known only after phase 1 when the buffer is sized to fit).
// With `comp` known and segments short enough for the register kernel the
// records are placed by the encode kernel itself (`direct`).
NzEncItem enc_item(const NzGeom& g, const void* in, uint8_t* packed, uint8_t* ws, const EncLayout& L,
                   uint8_t* comp, uint64_t comp_cap, uint64_t* d_total, uint32_t* d_status,
                   uint32_t ns, uint8_t* norm) {
  NzEncItem it{};
  it.in = (const uint16_t*)in;
  it.packed = packed;
  it.ws = ws;
  it.comp = comp;
  it.comp_cap = comp_cap;
  it.d_total = d_total;
  it.d_status = d_status;
  it.nm = NzNorm{ns ? norm : nullptr, log2_of(ns ? ns : 1)};
  it.g = g;
  it.exps = L.exps;
  it.tab_ser = L.tab_ser;
  it.info = L.info;
  it.carry = L.carry;
  it.slots = L.slots;
  it.states = L.states;
  it.seg_words = L.seg_words;
  it.seg_sbytes = L.seg_sbytes;
  it.seg_units = L.seg_units;
  it.chunk_units = L.chunk_units;
  it.pub = L.pub;
  it.placed = L.placed;
  it.lb_state = L.lb_state;
  it.old_comp = nullptr;
  it.use_placed = 0;
  it.nonce = next_nonce();
  it.d_gave_up = nullptr;
  it.direct = (comp != nullptr && g.n_segs != 0 && enc_in_registers(g)) ? 1u : 0u;
  it.spin_limit = g_lookback_spins.load(std::memory_order_relaxed);
  return it;
}

// running totals of chunks and segments; false when they do not fit a grid
bool enc_batch_close(NzEncBatch* b) {
  uint64_t chunks = 0, segs = 0;
  for (uint32_t i = 0; i < b->count; ++i) {
    chunks += b->item[i].g.n_chunks;
    segs += b->item[i].g.n_segs;
    if (chunks > 0x7FFFFFFFull || segs > 0x7FFFFFFFull) return false;
    b->item[i].chunk_end = (uint32_t)chunks;
    b->item[i].seg_end = (uint32_t)segs;
  }
  return true;
}

// One encode launch for the tensors of `b` whose segments are of class `cls`
// (0..3: up to 64 / 128 / 256 / 288 symbols per lane, coded from registers; 4: longer).
// The register encode kernels may use more than 64 KiB of LDS per workgroup
// (word staging): that has to be allowed once per kernel and device, and is
// done for all of them before the first encode on a device.
int allow_encode_lds() {
  static std::atomic<uint64_t> allowed{0};  // bit d: done on device d
  int dev = 0;
  NZ_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return fail(NZ_ERR_ARG, "device index out of range");
  if ((allowed.load(std::memory_order_acquire) >> dev) & 1ull) return NZ_OK;
  NZ_HIP(nz_allow_encode_lds<7>());
  NZ_HIP(nz_allow_encode_lds<3>());
  NZ_HIP(nz_allow_encode_lds<1>());
  NZ_HIP(nz_allow_encode_lds<0>());
  allowed.fetch_or(1ull << dev, std::memory_order_release);
  return NZ_OK;
}

// Words of LDS staging per wavefront for a direct encode of class `cls` with
// workgroups of `waves` wavefronts: what a workgroup can have without lowering
// the number of workgroups that the registers allow per compute unit (4, 6, 8
// wavefronts per SIMD unit for 256 and more, 128, 64 symbols per lane), less the
// kernel's own LDS.
uint32_t stage_words_for(int cls, uint32_t waves) {
  const uint32_t waves_per_cu = cls >= 2 ? 16u : cls == 1 ? 24u : 32u;
  const uint32_t groups = waves_per_cu / waves ? waves_per_cu / waves : 1u;
  const uint32_t per_group = 160u * 1024u / groups;
  const uint32_t fixed = ((uint32_t)sizeof(NzEncLds) + 511u) & ~511u;  // the kernel's own LDS
  if (per_group <= fixed + 1024u) return 0;
  const uint32_t per_wave = ((per_group - fixed - 512u) / waves) & ~127u;  // bytes (512: the closing slack, rounding)
  return per_wave / 2;
}

template <int S>
int launch_encode_class(NzEncBatch& b, int cls, uint32_t chunks, uint32_t max_spc, hipStream_t st) {
  const uint32_t waves = max_spc < 4 ? 4 : max_spc;
  const dim3 grid(chunks), block(64 * waves);
  bool direct = false;
  for (uint32_t i = 0; i < b.count; ++i) direct = direct || b.item[i].direct;
  b.stage_words = (direct && cls < 4) ? stage_words_for(cls, waves) : 0u;
  const uint32_t lds = b.stage_words ? waves * b.stage_words * 2u + 16u : 0u;
  nz_launch_encode<S>(b, cls, grid, block, lds, st);
  return NZ_OK;
}

int enc_class(const NzGeom& g) {
  return g.lane_syms <= 64 ? 0 : g.lane_syms <= 128 ? 1 : g.lane_syms <= 256 ? 2 : g.lane_syms <= NZ_ENC_MAX_LANE_SYMS ? 3 : 4;
}

// Phase 1 for all tensors of the batch: everything up to the directory.  Header
// + directory land in each item's `hdr`, the container size in its *d_total.
int encode_phase1(NzEncBatch* b, int precision, uint32_t ns, hipStream_t st) {
  if (!enc_batch_close(b)) return fail(NZ_ERR_ARG, "too many chunks for one launch");
  if (int rc = allow_encode_lds()) return rc;
  for (uint32_t i = 0; i < b->count; ++i)
    if (int rc = launch_absmax(b->item[i].in, b->item[i].g.n, ns, const_cast<uint8_t*>(b->item[i].nm.bytes), st))
      return rc;
  // the tensors of the batch, by segment-length class: one launch per class in use
  for (int cls = 0; cls < 5; ++cls) {
    NzEncBatch sub{};
    uint32_t chunks = 0, max_spc = 1;
    for (uint32_t i = 0; i < b->count; ++i) {
      const NzEncItem& it = b->item[i];
      if (it.g.n_chunks == 0 || enc_class(it.g) != cls) continue;
      NzEncItem& d = sub.item[sub.count++];
      d = it;
      chunks += (uint32_t)it.g.n_chunks;
      d.chunk_end = chunks;
      if (it.g.spc > max_spc) max_spc = it.g.spc;
    }
    if (!sub.count) continue;
    int rc;
    switch (precision) {
      case 7: rc = launch_encode_class<7>(sub, cls, chunks, max_spc, st); break;
      case 3: rc = launch_encode_class<3>(sub, cls, chunks, max_spc, st); break;
      case 1: rc = launch_encode_class<1>(sub, cls, chunks, max_spc, st); break;
      default: rc = launch_encode_class<0>(sub, cls, chunks, max_spc, st); break;
    }
    if (rc) return rc;
  }
  NZ_HIP(hipGetLastError());
  return NZ_OK;
}

// Container sizes (and status) of the batch on the device, before the records
// are placed: for a caller that sizes the container's memory to fit.  Also
// writes the header-only container of a tensor without elements.
int encode_totals(NzEncBatch* b, hipStream_t st) {
  if (b->count) hipLaunchKernelGGL(nz_total_kernel, dim3(b->count), dim3(256), 0, st, *b);
  NZ_HIP(hipGetLastError());
  return NZ_OK;
}

// Phase 2: header, directory and records go to each item's `comp`; the
// container size lands in *d_total, bit 0 of *d_status is set when it does not fit.
int encode_phase2(NzEncBatch* b, hipStream_t st) {
  NzEncBatch rest{};  // what the encode kernel has not placed itself
  bool empty = false;  // a tensor without segments has no workgroup to write its header
  for (uint32_t i = 0; i < b->count; ++i) {
    empty = empty || b->item[i].g.n_segs == 0;
    if (!b->item[i].direct) rest.item[rest.count++] = b->item[i];
  }
  if (empty)
    if (int rc = encode_totals(b, st)) return rc;
  if (!enc_batch_close(&rest)) return fail(NZ_ERR_ARG, "too many chunks for one launch");
  const uint32_t segs = rest.count ? rest.item[rest.count - 1].seg_end : 0;
  if (segs) {
    hipLaunchKernelGGL(nz_compact_kernel, dim3(segs), dim3(256), 0, st, rest);
    NZ_HIP(hipGetLastError());
  }
  return NZ_OK;
}

// The records of item i again, by nz_compact_kernel from what the encode kernel
// left in the scratch (into another buffer, or after a chunk gave up waiting).
// `placed_in`: the container the direct encode wrote to (records that went there
// from LDS exist nowhere else and are copied from it).
int encode_replace(const NzEncItem& item, const uint8_t* placed_in, hipStream_t st) {
  NzEncBatch one{};
  one.count = 1;
  one.item[0] = item;
  one.item[0].use_placed = item.direct;
  one.item[0].old_comp = placed_in;
  one.item[0].direct = 0;
  return encode_phase2(&one, st);
}

// `flags`: NZ_DECODE_STREAM_OUT / NZ_DECODE_RESIDENT_OUT override the output
// policy that is otherwise chosen by the size of the dense tensor
int decode_launch(const NzGeom& g, int precision, const void* comp, uint64_t comp_bytes,
                  const void* packed, void* out, uint32_t* d_status, uint32_t ns, const void* norm,
                  int flags, hipStream_t st) {
  if (g.n_chunks == 0) return NZ_OK;
  const NzNorm nm{ns ? (const uint8_t*)norm : nullptr, log2_of(ns ? ns : 1)};
  const uint32_t so = (flags & NZ_DECODE_STREAM_OUT) ? 1u : (flags & NZ_DECODE_RESIDENT_OUT) ? 0u
                                                                                              : (nz_stream_output(g.n) ? 1u : 0u);
  switch (precision) {
    case 7: nz_launch_decode<7>(g, comp, comp_bytes, packed, out, d_status, nm, so, st); break;
    case 3: nz_launch_decode<3>(g, comp, comp_bytes, packed, out, d_status, nm, so, st); break;
    case 1: nz_launch_decode<1>(g, comp, comp_bytes, packed, out, d_status, nm, so, st); break;
    default: nz_launch_decode<0>(g, comp, comp_bytes, packed, out, d_status, nm, so, st); break;
  }
  NZ_HIP(hipGetLastError());
  return NZ_OK;
}

// all items of one launch share the output policy (`stream_out`)
int decode_batch_launch(const NzBatch& b, uint32_t grid, uint32_t max_spc, int precision, bool stream_out,
                        uint32_t* d_status, hipStream_t st) {
  if (grid == 0) return NZ_OK;
  switch (precision) {
    case 7: nz_launch_decode_batch<7>(b, grid, max_spc, stream_out, d_status, st); break;
    case 3: nz_launch_decode_batch<3>(b, grid, max_spc, stream_out, d_status, st); break;
    case 1: nz_launch_decode_batch<1>(b, grid, max_spc, stream_out, d_status, st); break;
    default: nz_launch_decode_batch<0>(b, grid, max_spc, stream_out, d_status, st); break;
  }
  NZ_HIP(hipGetLastError());
  return NZ_OK;
}

int gemv_launch(const NzBatch& b, uint32_t grid, uint32_t max_spc, int precision, uint32_t* d_status,
                hipStream_t st) {
  switch (precision) {
    case 7: nz_launch_gemv<7>(b, grid, max_spc, d_status, st); break;
    case 3: nz_launch_gemv<3>(b, grid, max_spc, d_status, st); break;
    case 1: nz_launch_gemv<1>(b, grid, max_spc, d_status, st); break;
    default: nz_launch_gemv<0>(b, grid, max_spc, d_status, st); break;
  }
  NZ_HIP(hipGetLastError());
  return NZ_OK;
}

int make_geom(NzGeom* g, uint64_t n, uint32_t chunk, uint32_t lane_syms) {
  if (nz_geom_make(g, n, chunk, lane_syms))
    return fail(NZ_ERR_ARG,
                "unsupported geometry: lane_syms must be a multiple of 8 (>= 16), chunk_size a multiple "
                "of 512 cut into 1..8 segments of 64*lane_syms, the last one at least 1024 long");
  if (g->n_chunks > 0x7FFFFFFFull) return fail(NZ_ERR_ARG, "tensor too large");
  return NZ_OK;
}

// nz_encode and nz_encode_static behind their argument checks: the three encode
// launches with `ws` as scratch.  Nothing here allocates or synchronises.
int encode_stateless(const void* dev_bf16, uint64_t n, int precision, uint32_t chunk_size, uint32_t lane_syms,
                     void* dev_packed, void* dev_comp, uint64_t comp_cap, uint8_t* ws, uint64_t ws_bytes,
                     const char* ws_error, uint64_t* dev_total, uint32_t* dev_status, uint32_t normalizer_size,
                     void* dev_norm, hipStream_t st, NzEncItem* item_out = nullptr) {
  if (!precision_ok(precision)) return fail(NZ_ERR_ARG, "precision must be one of 0, 1, 3, 7");
  if (!normalizer_ok(normalizer_size))
    return fail(NZ_ERR_ARG, "normalizer_size must be 0 or a power of two up to 1024");
  if (normalizer_size && n && (!dev_norm || ((uintptr_t)dev_norm & 7)))
    return fail(NZ_ERR_ARG, "normalizer bytes: null or not 8-byte aligned");
  NzGeom g;
  if (int rc = make_geom(&g, n, chunk_size, lane_syms)) return rc;
  if (!dev_comp || !dev_total || !dev_status || (n && (!dev_bf16 || !dev_packed)))
    return fail(NZ_ERR_ARG, "null pointer");
  if ((uintptr_t)dev_bf16 & 15) return fail(NZ_ERR_ALIGN, "dense input must be 16-byte aligned");
  if (((uintptr_t)dev_packed & 7) || ((uintptr_t)dev_comp & 15))
    return fail(NZ_ERR_ALIGN, "packed/comp buffers must be 8/16-byte aligned");
  const EncLayout L = enc_layout(g);
  if (ws_bytes < L.bytes) return fail(NZ_ERR_CAPACITY, ws_error);
  if (comp_cap < nz_geom_bound(&g)) return fail(NZ_ERR_CAPACITY, "dev_comp smaller than nz_exp_bound_bytes");
  NzEncBatch b{};
  b.count = 1;
  b.item[0] = enc_item(g, dev_bf16, (uint8_t*)dev_packed, ws, L, (uint8_t*)dev_comp, comp_cap, dev_total, dev_status,
                       normalizer_size, (uint8_t*)dev_norm);
  if (item_out) *item_out = b.item[0];
  if (int rc = encode_phase1(&b, precision, normalizer_size, st)) return rc;
  return encode_phase2(&b, st);
}

// Scratch of nz_encode_static: device memory that exists from the moment the
// code object is loaded, one copy per GPU, so that the call allocates nothing.
// In host code `nz_static_scratch` is only a handle for hipGetSymbolAddress;
// the device address of each GPU's copy is looked up once and kept.
static __device__ __align__(256) uint8_t nz_static_scratch[NZ_STATIC_SCRATCH_BYTES];
#define NZ_MAX_DEVICES 64
std::mutex g_static_mu;
uint8_t* g_static_ptr[NZ_MAX_DEVICES];

int static_scratch(uint8_t** out) {
  int dev = 0;
  NZ_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= NZ_MAX_DEVICES) return fail(NZ_ERR_ARG, "device index out of range");
  std::lock_guard<std::mutex> lock(g_static_mu);
  if (!g_static_ptr[dev]) {
    void* p = nullptr;
    NZ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(nz_static_scratch)));
    if (!p) return fail(NZ_ERR_HIP, "hipGetSymbolAddress returned a null address");
    g_static_ptr[dev] = (uint8_t*)p;
  }
  *out = g_static_ptr[dev];
  return NZ_OK;
}

// Stored exponent bytes (container + what the packed stream saves) of a tensor
// of n elements over the order-0 entropy of its exponents, as a function of
// the geometry: every lane and segment costs about 4.5 bits (its coder state
// less the 16 carried bits) and every segment a directory entry and padding
// (43 bytes a segment in all, a short last segment as much as a full one),
// every chunk a table (25 bytes), every tensor a header and a ragged end (up to
// ~190 bytes).  Fitted to measurements on N(0, 0.02) weights (2.545 bits per
// exponent: 1 byte of container is 3.14 symbols' worth of entropy), where it is
// within 0.0003 from a million elements up and within 0.0001 from 16 million:
//   58.7 M elements  131072/256 1.0096, 135168/264 1.0094, 131072/344 1.0076, 262144/512 1.0053
//   1 Mi elements    131072/256 1.0099, 139264/272 1.0098, 147456/288 1.0093, 262144/512 1.0056
//   (earlier fits, large tensors: 65536/256 1.0102, 65536/128 1.0185, 32768/64 1.036).
double est_ratio(uint64_t n, uint32_t chunk_syms, uint32_t lane_syms) {
  if (n == 0) return 1.0;
  const uint64_t seg = (uint64_t)lane_syms * NZ_LANES;
  const uint64_t full = n / chunk_syms, rest = n % chunk_syms;
  const uint64_t segs = full * ((chunk_syms + seg - 1) / seg) + (rest + seg - 1) / seg;
  const uint64_t chunks = full + (rest ? 1 : 0);
  return 1.0008 + (134.4 * (double)segs + 78.0 * (double)chunks + 600.0) / (double)n;
}

// The overhead is a fixed number of bytes, so the ratio grows as the entropy
// shrinks (weights drift while they are trained: a 1024 x 1024 GPT-2 weight
// gained 0.00015 in 20 AdamW steps): a geometry counts as inside a budget when
// its estimate leaves 0.0003 in hand.
bool in_budget(uint64_t n, uint32_t chunk_syms, uint32_t lane_syms, double budget) {
  return est_ratio(n, chunk_syms, lane_syms) + 0.0003 <= budget;
}

// The geometry a manager uses for a tensor of n elements when the caller
// leaves the segment length to the library.  The library's own chunk: eight
// segments per chunk, from the default 256 symbols per lane up to 512 in steps
// of 8, the shortest (most wavefronts) that is inside the budget.  A given
// chunk: the shortest valid segments from 256 symbols per lane up that are
// inside it.  A tensor too small for any of these to reach the budget (its
// header alone is above it) keeps the starting point: its bytes do not matter
// and its decode time does.
void default_geometry(uint64_t n, bool own_chunk, double budget, uint32_t* chunk_syms, uint32_t* lane_syms) {
  if (own_chunk) {
    *chunk_syms = NZ_DEFAULT_CHUNK;
    *lane_syms = NZ_DEFAULT_LANE_SYMS;
    for (uint32_t lane = NZ_DEFAULT_LANE_SYMS; lane <= 512; lane += 8) {
      const uint32_t chunk = lane * NZ_LANES * NZ_MAX_SEGS_PER_CHUNK;
      if (!in_budget(n, chunk, lane, budget)) continue;
      *chunk_syms = chunk;
      *lane_syms = lane;
      return;
    }
    return;
  }
  const uint32_t chunk = *chunk_syms;
  uint32_t first = 0, shortest = 0;
  for (uint32_t lane = 16; lane <= 65536; lane += 8) {
    if (nz_geom_check(chunk, lane)) continue;
    if (!shortest) shortest = lane;
    if (lane < NZ_DEFAULT_LANE_SYMS) continue;
    if (!first) first = lane;
    if (in_budget(n, chunk, lane, budget)) {
      *lane_syms = lane;
      return;
    }
  }
  // nothing fits the budget (a small tensor), or the chunk is too short for 256 symbols per lane
  *lane_syms = first ? first : (shortest ? shortest : NZ_DEFAULT_LANE_SYMS);
}

// a tensor large enough for the per-tensor terms of the estimate to vanish: what
// a manager reports as its nominal geometry before it has seen a tensor
constexpr uint64_t NZ_NOMINAL_N = 1ull << 28;

struct Entry {
  void* comp = nullptr;
  uint64_t comp_bytes = 0, comp_cap = 0;
  void* packed = nullptr;
  uint64_t packed_bytes = 0, packed_cap = 0;
  uint64_t n = 0;
  int dtype = NZ_DTYPE_BF16;
  uint32_t lane_syms = 0;  // geometry this entry was written with
  uint32_t chunk_syms = 0;
  void* norm = nullptr;    // one byte per normalizer group (managers with normalizer_size > 0)
  uint64_t norm_bytes = 0, norm_cap = 0;
  int pending = -1;        // rewrite slot whose result (container size) the host has not looked at yet
};

// One batch of in-place rewrites in flight: tensors written again under handles
// that already hold a tensor of the same size are encoded straight into the
// buffers they have, without allocation and without waiting for the container
// size.  The size comes back through pinned memory behind an event and is
// looked at when the entry is used next (or when the slot is needed again).
struct RewriteSlot {
  bool busy = false;
  hipEvent_t ev = nullptr;
  hipStream_t stream = nullptr;
  void* ws = nullptr;
  uint64_t ws_bytes = 0;
  uint64_t* d_totals = nullptr;  // 16 sizes, then 16 give-up marks (the nonce of the item that gave up): pinned host
                                 // memory, this is its address on the device ...
  uint64_t* h_totals = nullptr;  // ... and this the one on the host
  uint32_t count = 0;
  std::string names[NZ_ENC_BATCH_MAX];
  NzEncBatch b;
};

}  // namespace

struct nz_manager {
  int precision;
  uint32_t normalizer = 0;  // elements per normalizer group, 0 = none
  uint32_t chunk_syms, lane_syms;
  bool own_chunk = false;   // chunk_size 0 was given: the library's own table scope
  bool own_lanes = false;   // lane_syms 0 or AUTO was given: the segment length follows the size budget
  bool auto_lanes = false;  // pick the geometry per tensor so that small tensors still fill the GPU
  double budget = NZ_DEFAULT_SIZE_BUDGET;  // stored exponent bytes over their order-0 entropy the manager's own choices stay within
  hipStream_t last_stream = nullptr;  // stream of the last call that used the shared scratch (write, product, row gather)
  bool has_stream = false;
  hipEvent_t order_ev = nullptr;      // orders such a call on another stream behind it
  uint32_t given_chunk = 0;  // the caller's chunk_size (0: the library's own)
  uint32_t slots = 768;     // decode workgroups of eight wavefronts the device holds at once (3 per CU)
  std::unordered_map<std::string, Entry> entries;  // compress_cache + meta_cache
  std::unordered_map<std::string, std::pair<uint32_t, uint32_t>> hints;  // name -> (chunk, lane) for its next writes
  std::mutex mu;
  void* ws = nullptr;
  uint64_t ws_bytes = 0;
  uint32_t* d_status = nullptr;  // 256 bytes: decode status | container sizes and status words of a write batch
  uint64_t* h_pin = nullptr;     // pinned, 256 bytes: [0..15] those sizes, [16] decode status, [17..24] those status words
  long long* gemv_acc = nullptr;  // row accumulators of the matrix-vector product (all zero between calls)
  uint64_t gemv_rows = 0;         // rows the accumulator buffer can hold
  RewriteSlot rw[2];              // in-place rewrites in flight (two batches: the host runs one ahead)
  uint32_t rw_next = 0;
  // statistics: batches rewritten in place / entries that outgrew their buffer / entries whose records were
  // placed a second time because a chunk gave up waiting
  uint64_t rewrites = 0, rewrites_replaced = 0, rewrites_redone = 0;
};

extern "C" {

int nz_abi_version(void) { return 4; }

const char* nz_last_error(void) { return g_err.c_str(); }

uint64_t nz_packed_bytes(uint64_t n, int precision) { return nz_packed_bytes_of(n, precision); }

uint64_t nz_packed_stored_bytes(uint64_t n, int precision, uint32_t chunk_size, uint32_t lane_syms) {
  NzGeom g;
  if (nz_geom_make(&g, n, chunk_size, lane_syms)) return 0;
  return nz_packed_stored_bytes_of(&g, precision);
}

uint64_t nz_exp_bound_bytes(uint64_t n, uint32_t chunk_size, uint32_t lane_syms) {
  NzGeom g;
  if (nz_geom_make(&g, n, chunk_size, lane_syms)) return 0;
  return nz_geom_bound(&g);
}

uint64_t nz_encode_workspace_bytes(uint64_t n, uint32_t chunk_size, uint32_t lane_syms) {
  NzGeom g;
  if (nz_geom_make(&g, n, chunk_size, lane_syms)) return 0;
  return enc_layout(g).bytes;
}

uint64_t nz_norm_bytes(uint64_t n, uint32_t normalizer_size) {
  return normalizer_ok(normalizer_size) ? norm_bytes_of(n, normalizer_size) : 0;
}

int nz_split(const void* dev_bf16, uint64_t n, void* dev_exponents, void* dev_fractions,
             uint32_t normalizer_size, void* dev_norm, void* stream) {
  if (!normalizer_ok(normalizer_size))
    return fail(NZ_ERR_ARG, "normalizer_size must be 0 or a power of two up to 1024");
  if (n == 0) return NZ_OK;
  if (!dev_bf16 || !dev_exponents || !dev_fractions || (normalizer_size && !dev_norm))
    return fail(NZ_ERR_ARG, "null pointer");
  if (normalizer_size && ((uintptr_t)dev_norm & 7))
    return fail(NZ_ERR_ALIGN, "normalizer bytes must be 8-byte aligned");
  if (((uintptr_t)dev_bf16 & 15) || ((uintptr_t)dev_exponents & 7) || ((uintptr_t)dev_fractions & 7))
    return fail(NZ_ERR_ALIGN, "nz_split: pointers must be 16-byte (input) / 8-byte (outputs) aligned");
  const uint64_t blocks = (n + 2047) / 2048;
  if (blocks > 0x7FFFFFFFull) return fail(NZ_ERR_ARG, "tensor too large");
  if (int rc = launch_absmax(dev_bf16, n, normalizer_size, (uint8_t*)dev_norm, (hipStream_t)stream)) return rc;
  const NzNorm nm{normalizer_size ? (const uint8_t*)dev_norm : nullptr, log2_of(normalizer_size ? normalizer_size : 1)};
  hipLaunchKernelGGL(nz_split_unpacked_kernel, dim3((uint32_t)blocks), dim3(256), 0,
                     (hipStream_t)stream, (const uint16_t*)dev_bf16, n, (uint8_t*)dev_exponents,
                     (uint8_t*)dev_fractions, nm);
  NZ_HIP(hipGetLastError());
  return NZ_OK;
}

int nz_encode(const void* dev_bf16, uint64_t n, int precision, uint32_t chunk_size,
              uint32_t lane_syms, void* dev_packed, void* dev_comp, uint64_t comp_cap,
              void* dev_workspace, uint64_t workspace_bytes, uint64_t* dev_total,
              uint32_t* dev_status, uint64_t* host_total, uint32_t normalizer_size, void* dev_norm,
              void* stream) {
  if (!dev_workspace) return fail(NZ_ERR_ARG, "null pointer");
  if ((uintptr_t)dev_workspace & 255) return fail(NZ_ERR_ALIGN, "workspace must be 256-byte aligned");
  NzEncItem item;
  if (int rc = encode_stateless(dev_bf16, n, precision, chunk_size, lane_syms, dev_packed, dev_comp, comp_cap,
                                (uint8_t*)dev_workspace, workspace_bytes, "workspace too small", dev_total,
                                dev_status, normalizer_size, dev_norm, (hipStream_t)stream, &item))
    return rc;
  if (host_total) {
    hipStream_t st = (hipStream_t)stream;
    uint32_t hs = 0;
    NZ_HIP(hipMemcpyAsync(host_total, dev_total, 8, hipMemcpyDeviceToHost, st));
    NZ_HIP(hipMemcpyAsync(&hs, dev_status, 4, hipMemcpyDeviceToHost, st));
    NZ_HIP(hipStreamSynchronize(st));
    if (hs & 4u) {
      // a chunk gave up waiting for the sizes before it: the records once more, by the compaction
      if (int rc = encode_replace(item, item.comp, st)) return rc;
      NZ_HIP(hipMemcpyAsync(host_total, dev_total, 8, hipMemcpyDeviceToHost, st));
      NZ_HIP(hipMemcpyAsync(&hs, dev_status, 4, hipMemcpyDeviceToHost, st));
      NZ_HIP(hipStreamSynchronize(st));
    }
    if (hs & 1u) return fail(NZ_ERR_CAPACITY, "encoded container exceeds the output capacity");
  }
  return NZ_OK;
}

void nz_set_lookback_spins(uint32_t spins) { g_lookback_spins.store(spins, std::memory_order_relaxed); }

int nz_encode_static(const void* dev_bf16, uint64_t n, int precision, uint32_t chunk_size,
                     uint32_t lane_syms, void* dev_packed, void* dev_comp, uint64_t comp_cap,
                     uint64_t* dev_total, uint32_t* dev_status, uint32_t normalizer_size, void* dev_norm,
                     void* stream) {
  uint8_t* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  return encode_stateless(dev_bf16, n, precision, chunk_size, lane_syms, dev_packed, dev_comp, comp_cap, ws,
                          NZ_STATIC_SCRATCH_BYTES,
                          "tensor too large for nz_encode_static: its encode scratch exceeds NZ_STATIC_SCRATCH_BYTES",
                          dev_total, dev_status, normalizer_size, dev_norm, (hipStream_t)stream);
}

int nz_decode(const void* dev_comp, uint64_t comp_bytes, const void* dev_packed, uint64_t n,
              int precision, uint32_t chunk_size, uint32_t lane_syms, void* dev_bf16_out,
              uint32_t* dev_status, int flags, uint32_t normalizer_size, const void* dev_norm,
              void* stream) {
  const int check = flags & NZ_DECODE_CHECK;
  if (!precision_ok(precision)) return fail(NZ_ERR_ARG, "precision must be one of 0, 1, 3, 7");
  if (!normalizer_ok(normalizer_size))
    return fail(NZ_ERR_ARG, "normalizer_size must be 0 or a power of two up to 1024");
  if (normalizer_size && n && (!dev_norm || ((uintptr_t)dev_norm & 7)))
    return fail(NZ_ERR_ARG, "normalizer bytes: null or not 8-byte aligned");
  NzGeom g;
  if (int rc = make_geom(&g, n, chunk_size, lane_syms)) return rc;
  if (n == 0) return NZ_OK;
  if (!dev_comp || !dev_packed || !dev_bf16_out) return fail(NZ_ERR_ARG, "null pointer");
  if ((uintptr_t)dev_bf16_out & 15) return fail(NZ_ERR_ALIGN, "dense output must be 16-byte aligned");
  if (((uintptr_t)dev_comp & 15) || ((uintptr_t)dev_packed & 7))
    return fail(NZ_ERR_ALIGN, "comp/packed buffers must be 16/8-byte aligned");
  if (!dev_status) return fail(NZ_ERR_ARG, "dev_status is required (the kernel reports there)");
  if (comp_bytes < g.rec_off + NZ_TAIL_PAD) return fail(NZ_ERR_CORRUPT, "container shorter than its directory");
  hipStream_t st = (hipStream_t)stream;
  if ((flags & NZ_DECODE_STREAM_OUT) && (flags & NZ_DECODE_RESIDENT_OUT))
    return fail(NZ_ERR_ARG, "NZ_DECODE_STREAM_OUT and NZ_DECODE_RESIDENT_OUT exclude each other");
  if (int rc = decode_launch(g, precision, dev_comp, comp_bytes, dev_packed, dev_bf16_out, dev_status,
                             normalizer_size, dev_norm, flags, st))
    return rc;
  if (check) {
    uint32_t hs = 0;
    NZ_HIP(hipMemcpyAsync(&hs, dev_status, 4, hipMemcpyDeviceToHost, st));
    NZ_HIP(hipStreamSynchronize(st));
    if (hs) return fail(NZ_ERR_CORRUPT, "compressed container failed validation (status " + std::to_string(hs) + ")");
  }
  return NZ_OK;
}

// ---------------------------------------------------------------------------
// handle store
// ---------------------------------------------------------------------------

int nz_manager_create(int algorithm, int precision, int normalizer_size, uint32_t chunk_size,
                      uint32_t lane_syms, nz_manager** out) {
  if (!out) return fail(NZ_ERR_ARG, "null out pointer");
  if (algorithm != NZ_ALGO_ANS) return fail(NZ_ERR_ALGO, "Unsupported algorithm");
  if (!precision_ok(precision)) return fail(NZ_ERR_ARG, "precision must be one of 0, 1, 3, 7");
  if (normalizer_size < 0 || !normalizer_ok((uint32_t)normalizer_size))
    return fail(NZ_ERR_ARG, "normalizer_size must be 0 or a power of two up to 1024");
  const bool auto_lanes = lane_syms == NZ_LANE_SYMS_AUTO;
  const bool own_chunk = chunk_size == 0;
  const bool own_lanes = lane_syms == 0 || auto_lanes;
  if (own_chunk) {
    chunk_size = NZ_DEFAULT_CHUNK;
    // an explicit segment length too short for eight segments to cover the
    // default chunk goes with the smaller table scope
    if (!own_lanes && (uint64_t)lane_syms * NZ_LANES * NZ_MAX_SEGS_PER_CHUNK < chunk_size) chunk_size = 65536;
  }
  if (own_lanes) default_geometry(NZ_NOMINAL_N, own_chunk, NZ_DEFAULT_SIZE_BUDGET, &chunk_size, &lane_syms);
  NzGeom g;
  if (int rc = make_geom(&g, 0, chunk_size, lane_syms)) return rc;
  nz_manager* m = new nz_manager();
  m->precision = precision;
  m->normalizer = (uint32_t)normalizer_size;
  m->chunk_syms = chunk_size;
  m->own_chunk = own_chunk;
  m->own_lanes = own_lanes;
  m->given_chunk = own_chunk ? 0u : chunk_size;
  m->lane_syms = lane_syms;
  m->auto_lanes = auto_lanes;
  // device block and its pinned mirror, 1 KiB each: [0, 256) as described at the members;
  // [256 + 256 k, ...) the 16 container sizes of rewrite slot k; the last word a status sink
  hipError_t e = hipMalloc((void**)&m->d_status, 1024);
  if (e == hipSuccess) e = hipMemset(m->d_status, 0, 1024);
  if (e == hipSuccess) e = hipHostMalloc((void**)&m->h_pin, 1024, hipHostMallocDefault);
  // the sizes of a rewrite are written by the kernel straight into the pinned block (it is
  // mapped into the device's address space): no copy has to be enqueued to bring them back
  void* pin_dev = nullptr;
  if (e == hipSuccess) e = hipHostGetDevicePointer(&pin_dev, m->h_pin, 0);
  if (e == hipSuccess) std::memset(m->h_pin, 0, 1024);
  for (int k = 0; k < 2 && e == hipSuccess; ++k) {
    m->rw[k].d_totals = reinterpret_cast<uint64_t*>(reinterpret_cast<uint8_t*>(pin_dev) + 256 + 256 * k);
    m->rw[k].h_totals = reinterpret_cast<uint64_t*>(reinterpret_cast<uint8_t*>(m->h_pin) + 256 + 256 * k);
    e = hipEventCreateWithFlags(&m->rw[k].ev, hipEventDisableTiming);
  }
  if (e == hipSuccess) e = hipEventCreateWithFlags(&m->order_ev, hipEventDisableTiming);
  int dev = 0, cus = 0;
  if (e == hipSuccess) e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess && cus > 0) m->slots = 3u * (uint32_t)cus;
  if (e != hipSuccess) {
    for (int k = 0; k < 2; ++k)
      if (m->rw[k].ev) (void)hipEventDestroy(m->rw[k].ev);
    if (m->order_ev) (void)hipEventDestroy(m->order_ev);
    if (m->d_status) (void)hipFree(m->d_status);
    if (m->h_pin) (void)hipHostFree(m->h_pin);
    delete m;
    return fail(NZ_ERR_HIP, std::string("nz_manager_create: ") + hipGetErrorString(e));
  }
  *out = m;
  return NZ_OK;
}

void nz_manager_destroy(nz_manager* m) {
  if (!m) return;
  for (auto& kv : m->entries) {
    if (kv.second.comp) (void)hipFree(kv.second.comp);
    if (kv.second.packed) (void)hipFree(kv.second.packed);
    if (kv.second.norm) (void)hipFree(kv.second.norm);
  }
  if (m->ws) (void)hipFree(m->ws);
  for (int k = 0; k < 2; ++k) {
    if (m->rw[k].ws) (void)hipFree(m->rw[k].ws);
    if (m->rw[k].ev) (void)hipEventDestroy(m->rw[k].ev);
  }
  if (m->gemv_acc) (void)hipFree(m->gemv_acc);
  if (m->order_ev) (void)hipEventDestroy(m->order_ev);
  if (m->d_status) (void)hipFree(m->d_status);
  if (m->h_pin) (void)hipHostFree(m->h_pin);
  delete m;
}

double nz_estimated_size_ratio(uint64_t n, uint32_t chunk_size, uint32_t lane_syms) {
  if (nz_geom_check(chunk_size, lane_syms)) return 0.0;
  return est_ratio(n, chunk_size, lane_syms);
}

double nz_manager_size_budget(const nz_manager* m) { return m ? m->budget : 0.0; }

int nz_manager_in_budget(const nz_manager* m, uint64_t n, uint32_t chunk_size, uint32_t lane_syms) {
  return m && !nz_geom_check(chunk_size, lane_syms) && in_budget(n, chunk_size, lane_syms, m->budget) ? 1 : 0;
}

int nz_manager_set_size_budget(nz_manager* m, double ratio) {
  if (!m) return fail(NZ_ERR_ARG, "null manager");
  if (!(ratio > 1.002 && ratio <= 2.0)) return fail(NZ_ERR_ARG, "size budget must be above 1.002 and at most 2");
  std::lock_guard<std::mutex> lock(m->mu);
  m->budget = ratio;
  if (m->own_lanes) {
    uint32_t chunk = m->own_chunk ? 0u : m->given_chunk, lane = 0;
    default_geometry(NZ_NOMINAL_N, m->own_chunk, ratio, &chunk, &lane);
    if (nz_geom_check(chunk, lane)) return fail(NZ_ERR_ARG, "no valid geometry for this chunk size");
    m->chunk_syms = chunk;
    m->lane_syms = lane;
  }
  return NZ_OK;
}

}  // extern "C"

// ---- write: begin (everything up to the directory, on the device) | one host
// ---- synchronisation for the sizes | finish (exact-size buffer, compaction) ----

#define NZ_WRITE_BATCH_MAX 16

namespace {

struct PendingWrite {
  std::string name;
  Entry ent, old;
  NzGeom g;
  EncLayout L;
  uint8_t* ws = nullptr;
};

void release_entry(Entry& e) {
  if (e.comp) (void)hipFree(e.comp);
  if (e.packed) (void)hipFree(e.packed);
  if (e.norm) (void)hipFree(e.norm);
  e.comp = e.packed = e.norm = nullptr;
}

// Geometry of a tensor of n elements.  Throughput of both codec directions is
// set by the number of wavefronts in flight (one per 64 * lane_syms elements),
// the stored size by the number of segments (est_ratio).  A manager that was
// given a segment length uses it.  One that was not chooses per tensor: the
// shortest segments from the default up whose estimated size is inside the
// manager's budget (default_geometry: at the default budget of 1.01 that is
// 131072/256 from about six million elements up and 264 to 280 symbols per lane
// for the one to four million elements of a GPT-2 weight).  In auto mode a
// tensor too small to give every SIMD two wavefronts may get shorter segments
// still (and, with the library's own chunk, a table scope to match), but only
// inside the same budget: at 1.01 nothing shorter qualifies, so a small tensor
// keeps its size and is served well by the calls that take several tensors
// per launch; a caller who raises the budget buys wavefronts with bytes.
int pick_geometry(const nz_manager* m, const char* name, uint64_t n, NzGeom* g, uint32_t* chunk_out,
                  uint32_t* lane_out) {
  uint32_t lane_syms = m->lane_syms, chunk_syms = m->chunk_syms;
  const auto hint = m->hints.find(name);
  if (hint != m->hints.end()) {  // nz_manager_geometry_hint
    *chunk_out = hint->second.first;
    *lane_out = hint->second.second;
    return make_geom(g, n, *chunk_out, *lane_out);
  }
  if (m->own_lanes) default_geometry(n, m->own_chunk, m->budget, &chunk_syms, &lane_syms);
  if (m->auto_lanes && m->own_chunk) {
    // The device holds `slots` decode workgroups (three per compute unit) at
    // once, and a launch is fastest when every compute unit has the same number
    // of them: 378 workgroups on 256 units run as long as 512 would (measured on
    // a 4096 x 14336 matrix: 51 us with 378 chunks, 38 us with 512).  A tensor
    // with more chunks than slots keeps the geometry chosen above.  A smaller
    // one may be cut into one, two or three workgroups per compute unit (eight
    // segments of 64 to 512 symbols per lane each) when that is inside the size
    // budget and the model below promises 10 % or more; a tensor too small for
    // that may get 32 Ki chunks of eight 4 Ki segments (again: only inside the
    // budget).  Time of a round ~ symbols per lane x time of a step, which
    // grows with the wavefronts that share a SIMD unit (2, 4, 6 of them: about
    // 107, 147, 215 ns per step).
    const uint64_t slots = m->slots, cus = slots / 3;
    const uint64_t chunks = (n + chunk_syms - 1) / chunk_syms;
    if (chunks <= slots && cus != 0) {
      static const uint32_t step_ns[3] = {107, 147, 215};
      const uint64_t per_cu = chunks ? (chunks + cus - 1) / cus : 1;  // 1..3 workgroups per compute unit
      uint64_t best_t = (uint64_t)lane_syms * step_ns[per_cu - 1];
      bool found = false;
      for (uint32_t k = 1; k <= 3; ++k) {
        const uint64_t per_lane = (n + k * cus * 512 - 1) / (k * cus * 512);  // a chunk is 8 x 64 lanes
        const uint32_t lane = (uint32_t)((per_lane + 7) / 8) * 8;
        if (lane < 64 || lane > 512) continue;
        const uint32_t chunk = lane * NZ_LANES * NZ_MAX_SEGS_PER_CHUNK;
        if (nz_geom_check(chunk, lane) || !in_budget(n, chunk, lane, m->budget)) continue;
        const uint64_t t = (uint64_t)lane * step_ns[k - 1];
        if (10 * t < 9 * best_t) {  // another geometry only for a gain above 10 %
          best_t = t;
          lane_syms = lane;
          chunk_syms = chunk;
          found = true;
        }
      }
      if (!found && n < (uint64_t)64 * cus * 512 && in_budget(n, 32768, 64, m->budget)) {
        chunk_syms = 32768;
        lane_syms = 64;
      }
    }
  } else if (m->auto_lanes) {
    // a chunk size given by the caller: shorter segments while that is a valid
    // geometry inside the size budget and the tensor has fewer than 2048 segments
    while (lane_syms > 16 && nz_geom_check(chunk_syms, (lane_syms / 2 + 7) & ~7u) == 0 &&
           in_budget(n, chunk_syms, (lane_syms / 2 + 7) & ~7u, m->budget) &&
           n / ((uint64_t)lane_syms * NZ_LANES) < 2048)
      lane_syms = (lane_syms / 2 + 7) & ~7u;
  }
  *chunk_out = chunk_syms;
  *lane_out = lane_syms;
  return make_geom(g, n, chunk_syms, lane_syms);
}

// The manager's 256-byte device block: [0, 4) status of decode launches, [64, 192)
// container sizes of a write batch, [192, 256) its status words.
uint64_t* write_totals(nz_manager* m) { return reinterpret_cast<uint64_t*>(reinterpret_cast<uint8_t*>(m->d_status) + 64); }
uint32_t* write_status(nz_manager* m) { return reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(m->d_status) + 192); }

// Takes the entry `name` out of the store (cuda/high_level.cu:137-140: an existing
// entry is replaced; its buffers are reused when large enough, which also avoids
// a device-wide hipFree stall), allocates what has a known size and describes
// the tensor to the encode kernels (`item`; scratch slice `ws`, container size
// and status in slot `slot` of the manager's device block).
int write_begin(nz_manager* m, const char* name, const void* dev_data, uint64_t n, int dtype,
                uint32_t chunk_syms, uint32_t lane_syms, const NzGeom& g, uint8_t* ws, PendingWrite* pw,
                uint32_t slot, NzEncItem* item) {
  pw->name = name;
  pw->g = g;
  pw->L = enc_layout(g);
  pw->ws = ws;
  auto it = m->entries.find(name);
  if (it != m->entries.end()) {
    pw->old = it->second;
    m->entries.erase(it);
  }
  Entry& ent = pw->ent;
  Entry& old = pw->old;
  ent.n = n;
  ent.dtype = dtype;
  ent.lane_syms = lane_syms;
  ent.chunk_syms = chunk_syms;
  ent.packed_bytes = nz_packed_stored_bytes_of(&g, m->precision);
  ent.norm_bytes = norm_bytes_of(n, m->normalizer);
  hipError_t e = hipSuccess;
  if (ent.norm_bytes) {
    if (old.norm && old.norm_cap >= ent.norm_bytes && old.norm_cap <= ent.norm_bytes + 4096) {
      ent.norm = old.norm;
      ent.norm_cap = old.norm_cap;
      old.norm = nullptr;
    } else {
      ent.norm_cap = ent.norm_bytes + 8;
      e = hipMalloc(&ent.norm, ent.norm_cap);
    }
  }
  if (e == hipSuccess) {
    if (old.packed && old.packed_cap >= ent.packed_bytes && old.packed_cap <= ent.packed_bytes + 4096) {
      ent.packed = old.packed;
      ent.packed_cap = old.packed_cap;
      old.packed = nullptr;
    } else {
      ent.packed_cap = ent.packed_bytes ? ent.packed_bytes : 8;
      e = hipMalloc(&ent.packed, ent.packed_cap);
    }
  }
  if (e != hipSuccess) return fail(NZ_ERR_HIP, std::string("write: ") + hipGetErrorString(e));
  // where the container goes is decided once its size is known
  *item = enc_item(g, dev_data, (uint8_t*)ent.packed, ws, pw->L, nullptr, ~0ull, write_totals(m) + slot,
                   write_status(m) + slot, m->normalizer, (uint8_t*)ent.norm);
  return NZ_OK;
}

// With the container size known on the host: a buffer of that size for the records.
int write_place(PendingWrite* pw, uint64_t total, NzEncItem* item) {
  Entry& ent = pw->ent;
  Entry& old = pw->old;
  ent.comp_bytes = total;
  hipError_t e = hipSuccess;
  if (old.comp && old.comp_cap >= ent.comp_bytes && old.comp_cap <= ent.comp_bytes + ent.comp_bytes / 16 + 4096) {
    ent.comp = old.comp;
    ent.comp_cap = old.comp_cap;
    old.comp = nullptr;
  } else {
    // a little headroom: the next write of this handle (an optimizer step
    // later) is a few bytes longer or shorter and can reuse the buffer
    ent.comp_cap = ent.comp_bytes + ent.comp_bytes / 64 + 1024;
    e = hipMalloc(&ent.comp, ent.comp_cap);
  }
  if (e != hipSuccess) return fail(NZ_ERR_HIP, std::string("write: ") + hipGetErrorString(e));
  item->comp = (uint8_t*)ent.comp;
  item->comp_cap = ent.comp_cap;
  return NZ_OK;
}

// Look at the outcome of rewrite slot k (waiting for it only if it is still
// running): the container sizes become known, and an entry whose new container
// did not fit the buffer it had gets a larger one, filled by a second
// compaction from the slot's scratch, which nothing has touched since.
int settle_slot(nz_manager* m, int k) {
  RewriteSlot& s = m->rw[k];
  if (!s.busy) return NZ_OK;
  if (hipEventQuery(s.ev) != hipSuccess) NZ_HIP(hipEventSynchronize(s.ev));
  // the slot stays busy until every entry of the batch has been handled: a call that fails
  // half way leaves the others pending, and the next use of the slot or of such an entry tries again
  for (uint32_t j = 0; j < s.count; ++j) {
    auto it = m->entries.find(s.names[j]);
    if (it == m->entries.end() || it->second.pending != k) continue;
    Entry& ent = it->second;
    uint64_t total = s.h_totals[j];
    if (s.h_totals[16 + j] == s.b.item[j].nonce) {
      // a chunk gave up waiting for the sizes before it: the records once more, by the compaction
      if (int rc = encode_replace(s.b.item[j], s.b.item[j].comp, s.stream)) return rc;
      NZ_HIP(hipStreamSynchronize(s.stream));
      s.h_totals[16 + j] = 0;
      ++m->rewrites_redone;
      total = s.h_totals[j];
    }
    if (total > ent.comp_cap) {
      // outgrown: a buffer that fits, the records moved again
      void* bigger = nullptr;
      const uint64_t cap = total + total / 32 + 4096;
      NZ_HIP(hipMalloc(&bigger, cap));
      NzEncItem again = s.b.item[j];
      again.comp = (uint8_t*)bigger;
      again.comp_cap = cap;
      int rc = encode_replace(again, s.b.item[j].comp, s.stream);
      if (rc == NZ_OK && hipStreamSynchronize(s.stream) != hipSuccess) rc = fail(NZ_ERR_HIP, "settle: synchronize failed");
      if (rc != NZ_OK) {
        (void)hipFree(bigger);
        return rc;
      }
      (void)hipFree(ent.comp);
      ent.comp = bigger;
      ent.comp_cap = cap;
      ++m->rewrites_replaced;
    }
    ent.comp_bytes = total;
    ent.pending = -1;
  }
  s.busy = false;
  return NZ_OK;
}

int settle_entry(nz_manager* m, const Entry& ent) { return ent.pending >= 0 ? settle_slot(m, ent.pending) : NZ_OK; }

int settle_all(nz_manager* m) {
  for (int k = 0; k < 2; ++k)
    if (int rc = settle_slot(m, k)) return rc;
  return NZ_OK;
}

// Is `st` being captured into a graph?  (An error of the query is taken as "no".)
bool capturing(hipStream_t st) {
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &cap) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return cap != hipStreamCaptureStatusNone;
}

// A call that may allocate, wait on the host or look at an event from the host
// cannot be recorded into a graph: it is refused with a message, before it
// touches anything (the capture stays valid).
int refuse_under_capture(hipStream_t st, bool may_block, const char* what) {
  if (may_block && capturing(st))
    return fail(NZ_ERR_ARG, std::string(what) + ": the stream is being captured into a graph and this call may "
                                               "allocate or wait on the host; capture nz_encode / nz_decode, or reads "
                                               "and products of entries that no write is pending for");
  return NZ_OK;
}

// Writes, products and row gathers of one manager share its scratch memory
// (encode workspace, row accumulators): they are ordered on the device.  When
// such a call arrives on another stream than the one before it, the new stream
// is made to wait (an event, no host synchronisation) for what the other has
// been given so far.  Streams under capture are left alone: what a graph holds
// is ordered by the graph's owner.
int order_scratch_use(nz_manager* m, hipStream_t st) {
  if (capturing(st)) return NZ_OK;
  if (m->has_stream && m->last_stream != st && !capturing(m->last_stream)) {
    // (a stream that has gone into capture since its last call here is left alone: an event
    // recorded on it now would become part of its graph)
    if (hipEventRecord(m->order_ev, m->last_stream) == hipSuccess) {
      NZ_HIP(hipStreamWaitEvent(st, m->order_ev, 0));
    } else {
      // the stream of the call before is gone (destroyed by its owner): whatever it was given
      // has to be finished the slow way
      (void)hipGetLastError();
      NZ_HIP(hipDeviceSynchronize());
    }
  }
  m->last_stream = st;
  m->has_stream = true;
  return NZ_OK;
}

int grow_workspace(nz_manager* m, uint64_t bytes, hipStream_t st) {
  if (m->ws_bytes >= bytes) return NZ_OK;
  // the previous scratch may still be in use by kernels on the stream
  NZ_HIP(hipStreamSynchronize(st));
  if (m->ws) NZ_HIP(hipFree(m->ws));
  m->ws = nullptr;
  m->ws_bytes = 0;
  NZ_HIP(hipMalloc(&m->ws, bytes));
  m->ws_bytes = bytes;
  return NZ_OK;
}

}  // namespace

extern "C" {

int nz_manager_write_batch(nz_manager* m, const char* const* names, const void* const* dev_data,
                           const uint64_t* ns, uint32_t count, int dtype, void* stream) {
  if (!m || (count && (!names || !dev_data || !ns))) return fail(NZ_ERR_ARG, "null manager, names, data or sizes");
  if (dtype != NZ_DTYPE_BF16) return fail(NZ_ERR_DTYPE, "Unsupported data type");
  if (count > NZ_WRITE_BATCH_MAX) return fail(NZ_ERR_ARG, "at most 16 tensors per batch");
  hipStream_t st = (hipStream_t)stream;
  std::lock_guard<std::mutex> lock(m->mu);  // also guards the geometry hints read below
  // a write allocates, synchronises or (in place) looks at events from the host
  if (int rc = refuse_under_capture(st, true, "write")) return rc;
  if (int rc = order_scratch_use(m, st)) return rc;
  // check everything and size the scratch before anything is touched
  NzGeom g[NZ_WRITE_BATCH_MAX];
  uint32_t chunk[NZ_WRITE_BATCH_MAX], lane[NZ_WRITE_BATCH_MAX];
  uint64_t at[NZ_WRITE_BATCH_MAX + 1];
  at[0] = 0;
  for (uint32_t i = 0; i < count; ++i) {
    if (!names[i]) return fail(NZ_ERR_ARG, "null name");
    for (uint32_t j = 0; j < i; ++j)
      if (std::strcmp(names[i], names[j]) == 0) return fail(NZ_ERR_ARG, "a name appears twice in the batch");
    if (ns[i] && !dev_data[i]) return fail(NZ_ERR_ARG, "null data pointer");
    if ((uintptr_t)dev_data[i] & 15) return fail(NZ_ERR_ALIGN, "dense input must be 16-byte aligned");
    if (int rc = pick_geometry(m, names[i], ns[i], &g[i], &chunk[i], &lane[i])) return rc;
    at[i + 1] = at[i] + enc_layout(g[i]).bytes;
  }
  // ---- in place: every handle already holds a tensor of this size and geometry.  The new
  // streams go straight into the buffers the entries have (an optimizer step changes the
  // container size by a few bytes; a buffer has ~1.5 % of headroom): no allocation, no free,
  // no wait.  The sizes are looked at later (settle_slot), where an entry that has outgrown
  // its buffer is given a larger one.
  bool in_place = count > 0;
  for (uint32_t i = 0; i < count && in_place; ++i) {
    auto it = m->entries.find(names[i]);
    in_place = it != m->entries.end() && ns[i] != 0 && it->second.n == ns[i] && it->second.dtype == dtype &&
               it->second.chunk_syms == chunk[i] && it->second.lane_syms == lane[i] && it->second.comp != nullptr;
  }
  if (in_place) {
    // the slot is free once its previous batch has been looked at; an entry written
    // again while its last rewrite is still unseen is settled first
    const int k = (int)m->rw_next;
    if (int rc = settle_slot(m, k)) return rc;
    for (uint32_t i = 0; i < count; ++i)
      if (int rc = settle_entry(m, m->entries.find(names[i])->second)) return rc;
    RewriteSlot& s = m->rw[k];
    if (s.ws_bytes < at[count]) {
      if (s.ws) {
        NZ_HIP(hipStreamSynchronize(st));
        NZ_HIP(hipFree(s.ws));
      }
      s.ws = nullptr;
      s.ws_bytes = 0;
      NZ_HIP(hipMalloc(&s.ws, at[count]));
      s.ws_bytes = at[count];
    }
    s.b = NzEncBatch{};
    s.b.count = count;
    s.count = count;
    s.stream = st;
    uint32_t* status_sink = m->d_status + 255;  // the sizes tell the host everything it needs
    for (uint32_t i = 0; i < count; ++i) {
      Entry& ent = m->entries.find(names[i])->second;
      s.names[i] = names[i];
      s.b.item[i] = enc_item(g[i], dev_data[i], (uint8_t*)ent.packed, (uint8_t*)s.ws + at[i], enc_layout(g[i]),
                             (uint8_t*)ent.comp, ent.comp_cap, s.d_totals + i, status_sink, m->normalizer,
                             (uint8_t*)ent.norm);
      s.b.item[i].d_gave_up = s.d_totals + 16 + i;
    }
    if (int rc = encode_phase1(&s.b, m->precision, m->normalizer, st)) return rc;
    if (int rc = encode_phase2(&s.b, st)) return rc;
    NZ_HIP(hipEventRecord(s.ev, st));  // behind it the sizes and give-up marks are in the pinned block
    for (uint32_t i = 0; i < count; ++i) {
      Entry& ent = m->entries.find(names[i])->second;
      ent.pending = k;
      ent.comp_bytes = ent.comp_cap;  // an upper bound that keeps every access inside the buffer until the size is known
    }
    s.busy = true;
    m->rw_next ^= 1u;
    ++m->rewrites;
    return NZ_OK;
  }
  // ---- otherwise: new entries (or entries of another size), buffers sized to fit
  if (int rc = settle_all(m)) return rc;
  if (int rc = grow_workspace(m, at[count], st)) return rc;
  PendingWrite pw[NZ_WRITE_BATCH_MAX];
  int rc = NZ_OK;
  uint32_t begun = 0;
  NzEncBatch b{};
  for (; begun < count && rc == NZ_OK; ++begun)
    rc = write_begin(m, names[begun], dev_data[begun], ns[begun], dtype, chunk[begun], lane[begun], g[begun],
                     (uint8_t*)m->ws + at[begun], &pw[begun], begun, &b.item[begun]);
  b.count = count;
  // phase 1 of all tensors: one launch per kernel, then the one host
  // synchronisation of the batch for the container sizes
  uint64_t* h_totals = m->h_pin;
  uint32_t* h_status = reinterpret_cast<uint32_t*>(m->h_pin + 17);
  if (rc == NZ_OK && count) {
    hipError_t e = hipMemsetAsync(write_status(m), 0, 64, st);
    if (e != hipSuccess) rc = fail(NZ_ERR_HIP, std::string("write: ") + hipGetErrorString(e));
    if (rc == NZ_OK) rc = encode_phase1(&b, m->precision, m->normalizer, st);
    if (rc == NZ_OK) rc = encode_totals(&b, st);
    if (rc == NZ_OK) {
      e = hipMemcpyAsync(h_totals, write_totals(m), 8 * count, hipMemcpyDeviceToHost, st);
      if (e == hipSuccess) e = hipMemcpyAsync(h_status, write_status(m), 4 * count, hipMemcpyDeviceToHost, st);
      if (e == hipSuccess) e = hipStreamSynchronize(st);
      if (e != hipSuccess) rc = fail(NZ_ERR_HIP, std::string("size readback: ") + hipGetErrorString(e));
    }
    for (uint32_t i = 0; i < count && rc == NZ_OK; ++i)
      if (h_status[i] & 1u) rc = fail(NZ_ERR_CAPACITY, "container too large for its directory");
  }
  // phase 2: exact-size buffers, then one launch moves all records
  for (uint32_t i = 0; i < count && rc == NZ_OK; ++i) rc = write_place(&pw[i], h_totals[i], &b.item[i]);
  if (rc == NZ_OK && count) rc = encode_phase2(&b, st);
  if (rc == NZ_OK) {
    for (uint32_t i = 0; i < count; ++i) {
      m->entries.emplace(pw[i].name, pw[i].ent);
      pw[i].ent = Entry();  // now owned by the store
    }
  }
  // whatever did not make it into the store is released, old buffers in any case
  for (uint32_t i = 0; i < begun; ++i) {
    release_entry(pw[i].old);
    release_entry(pw[i].ent);
  }
  return rc;
}

int nz_manager_write(nz_manager* m, const char* name, const void* dev_data, uint64_t n, int dtype,
                     void* stream) {
  if (!m || !name) return fail(NZ_ERR_ARG, "null manager or name");
  return nz_manager_write_batch(m, &name, &dev_data, &n, 1, dtype, stream);
}

int nz_manager_read(nz_manager* m, const char* name, void* dev_out, uint64_t cap_elems,
                    void* stream) {
  if (!m || !name) return fail(NZ_ERR_ARG, "null manager or name");
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  if (it == m->entries.end()) return fail(NZ_ERR_NOT_FOUND, "Data not found");
  if (int rc = refuse_under_capture((hipStream_t)stream, it->second.pending >= 0, "read")) return rc;
  if (int rc = settle_entry(m, it->second)) return rc;
  const Entry& ent = it->second;
  if (cap_elems < ent.n) return fail(NZ_ERR_CAPACITY, "output smaller than the stored tensor");
  if (ent.n == 0) return NZ_OK;
  if (!dev_out) return fail(NZ_ERR_ARG, "null output pointer");
  if ((uintptr_t)dev_out & 15) return fail(NZ_ERR_ALIGN, "dense output must be 16-byte aligned");
  NzGeom g;
  if (int rc = make_geom(&g, ent.n, ent.chunk_syms, ent.lane_syms)) return rc;
  return decode_launch(g, m->precision, ent.comp, ent.comp_bytes, ent.packed, dev_out, m->d_status,
                       m->normalizer, ent.norm, 0, (hipStream_t)stream);
}

int nz_manager_read_batch(nz_manager* m, const char* const* names, void* const* dev_outs,
                          const uint64_t* cap_elems, uint32_t count, void* stream) {
  if (!m || (count && (!names || !dev_outs || !cap_elems)))
    return fail(NZ_ERR_ARG, "null manager, names, outputs or capacities");
  std::lock_guard<std::mutex> lock(m->mu);
  // validate everything before the first launch: a failed call decodes nothing
  {
    bool pending = false;
    for (uint32_t i = 0; i < count; ++i) {
      if (!names[i]) return fail(NZ_ERR_ARG, "null name");
      auto it = m->entries.find(names[i]);
      if (it == m->entries.end()) return fail(NZ_ERR_NOT_FOUND, "Data not found");
      pending = pending || it->second.pending >= 0;
    }
    if (int rc = refuse_under_capture((hipStream_t)stream, pending, "read_batch")) return rc;
  }
  for (uint32_t i = 0; i < count; ++i) {
    auto it = m->entries.find(names[i]);
    if (int rc = settle_entry(m, it->second)) return rc;
    const Entry& ent = it->second;
    if (cap_elems[i] < ent.n) return fail(NZ_ERR_CAPACITY, "output smaller than the stored tensor");
    if (ent.n && !dev_outs[i]) return fail(NZ_ERR_ARG, "null output pointer");
    if ((uintptr_t)dev_outs[i] & 15) return fail(NZ_ERR_ALIGN, "dense output must be 16-byte aligned");
  }
  NzBatch b;
  std::memset(&b, 0, sizeof(b));
  uint32_t grid = 0, max_spc = 1;
  bool streaming = false;
  auto flush = [&]() -> int {
    int rc = decode_batch_launch(b, grid, max_spc, m->precision, streaming, m->d_status, (hipStream_t)stream);
    b.count = 0;
    grid = 0;
    max_spc = 1;
    return rc;
  };
  // a launch has one output policy: the tensors small enough to stay in the
  // last-level cache first, then (rarely any) the ones written with streaming stores
  for (int pass = 0; pass < 2; ++pass) {
    streaming = pass == 1;
    for (uint32_t i = 0; i < count; ++i) {
      const Entry& ent = m->entries.find(names[i])->second;
      if (ent.n == 0 || nz_stream_output(ent.n) != streaming) continue;
      NzGeom g;
      if (int rc = make_geom(&g, ent.n, ent.chunk_syms, ent.lane_syms)) return rc;
      if (b.count == NZ_BATCH_MAX || (uint64_t)grid + g.n_chunks > 0x7FFFFFFFull)
        if (int rc = flush()) return rc;
      NzBatchItem& it = b.item[b.count++];
      it.comp = (const uint8_t*)ent.comp;
      it.comp_bytes = ent.comp_bytes;
      it.packed = (const uint8_t*)ent.packed;
      it.out = (uint16_t*)dev_outs[i];
      it.norm = (const uint8_t*)ent.norm;
      b.log2n = log2_of(m->normalizer ? m->normalizer : 1);
      it.g = g;
      grid += (uint32_t)g.n_chunks;
      it.chunk_end = grid;
      if (g.spc > max_spc) max_spc = g.spc;
    }
    if (b.count)
      if (int rc = flush()) return rc;
  }
  return NZ_OK;
}

int nz_manager_gemv_rows_batch(nz_manager* m, const char* const* names, uint32_t count, const void* dev_x,
                               uint32_t x_rows, uint32_t in_features, const void* const* dev_bias,
                               void* const* dev_y, void* stream) {
  if (!m || !names || !dev_y || !dev_x) return fail(NZ_ERR_ARG, "null manager, names, input or outputs");
  if (count == 0 || count > NZ_BATCH_MAX) return fail(NZ_ERR_ARG, "between 1 and 16 matrices per call");
  if (x_rows == 0 || x_rows > NZ_GEMV_MAX_ROWS) return fail(NZ_ERR_ARG, "between 1 and 8 activation rows per call");
  if (in_features == 0 || in_features % NZ_GROUP_SYMS)
    return fail(NZ_ERR_ARG, "in_features must be a multiple of 512");
  if ((uintptr_t)dev_x & 15) return fail(NZ_ERR_ALIGN, "activation must be 16-byte aligned");
  if (x_rows > 1 && m->normalizer)
    return fail(NZ_ERR_ARG, "several activation rows per call are not built for managers with normalizers");
  hipStream_t st = (hipStream_t)stream;
  std::lock_guard<std::mutex> lock(m->mu);
  NzBatch b;
  std::memset(&b, 0, sizeof(b));
  b.x = (const uint16_t*)dev_x;
  b.in_features = in_features;
  b.x_rows = x_rows;
  b.log2n = log2_of(m->normalizer ? m->normalizer : 1);
  // accumulator pairs per row of a matrix: as many as the kernel that serves x_rows holds per lane
  const uint32_t mr = x_rows <= 1 ? 1u : x_rows <= 2 ? 2u : x_rows <= 4 ? 4u : 8u;
  uint64_t grid = 0, rows = 0;
  uint32_t max_spc = 1;
  {
    bool blocks = false;
    uint64_t want_rows = 0;
    for (uint32_t i = 0; i < count; ++i) {
      if (!names[i]) return fail(NZ_ERR_ARG, "null name");
      auto it = m->entries.find(names[i]);
      if (it == m->entries.end()) return fail(NZ_ERR_NOT_FOUND, "Data not found");
      blocks = blocks || it->second.pending >= 0;
      want_rows += it->second.n / in_features * mr;
    }
    if (int rc = refuse_under_capture(st, blocks || m->gemv_rows < want_rows, "gemv_batch")) return rc;
    if (int rc = order_scratch_use(m, st)) return rc;
  }
  for (uint32_t i = 0; i < count; ++i) {
    auto it = m->entries.find(names[i]);
    if (int rc = settle_entry(m, it->second)) return rc;
    const Entry& ent = it->second;
    if (ent.n == 0 || ent.n % in_features)
      return fail(NZ_ERR_ARG, "stored tensor is not a matrix with rows of in_features elements");
    if (!dev_y[i] || ((uintptr_t)dev_y[i] & 1)) return fail(NZ_ERR_ARG, "null or misaligned output pointer");
    if (dev_bias && dev_bias[i] && ((uintptr_t)dev_bias[i] & 1)) return fail(NZ_ERR_ALIGN, "misaligned bias");
    NzGeom g;
    if (int rc = make_geom(&g, ent.n, ent.chunk_syms, ent.lane_syms)) return rc;
    NzBatchItem& bi = b.item[i];
    bi.comp = (const uint8_t*)ent.comp;
    bi.comp_bytes = ent.comp_bytes;
    bi.packed = (const uint8_t*)ent.packed;
    bi.norm = (const uint8_t*)ent.norm;
    bi.g = g;
    grid += g.n_chunks;
    bi.chunk_end = (uint32_t)grid;
    if (g.spc > max_spc) max_spc = g.spc;
    bi.bias = dev_bias ? (const uint16_t*)dev_bias[i] : nullptr;
    bi.y = (uint16_t*)dev_y[i];
    bi.reserved = (uint32_t)rows;  // first accumulator pair, turned into a pointer below
    rows += ent.n / in_features * mr;
    if (grid > 0x7FFFFFFFull || rows > 0x7FFFFFFFull) return fail(NZ_ERR_ARG, "batch too large");
  }
  if (m->gemv_rows < rows) {
    // the buffer in use may still be read by kernels on the stream
    NZ_HIP(hipStreamSynchronize(st));
    if (m->gemv_acc) NZ_HIP(hipFree(m->gemv_acc));
    m->gemv_acc = nullptr;
    m->gemv_rows = 0;
    const uint64_t want = rows < 65536 ? 65536 : rows;
    NZ_HIP(hipMalloc((void**)&m->gemv_acc, want * 16));
    NZ_HIP(hipMemset(m->gemv_acc, 0, want * 16));
    m->gemv_rows = want;
  }
  for (uint32_t i = 0; i < count; ++i) {
    b.item[i].acc = m->gemv_acc + 2 * (uint64_t)b.item[i].reserved;
    b.item[i].reserved = 0;
  }
  b.count = count;
  return gemv_launch(b, (uint32_t)grid, max_spc, m->precision, m->d_status, st);
}

int nz_manager_gemv_batch(nz_manager* m, const char* const* names, uint32_t count, const void* dev_x,
                          uint32_t in_features, const void* const* dev_bias, void* const* dev_y,
                          void* stream) {
  return nz_manager_gemv_rows_batch(m, names, count, dev_x, 1, in_features, dev_bias, dev_y, stream);
}

int nz_manager_gather_rows(nz_manager* m, const char* name, const void* dev_indices, uint64_t count,
                           uint32_t row_len, void* dev_out, void* stream) {
  if (!m || !name) return fail(NZ_ERR_ARG, "null manager or name");
  if (count == 0) return NZ_OK;
  if (!dev_indices || !dev_out) return fail(NZ_ERR_ARG, "null indices or output");
  if (((uintptr_t)dev_indices & 7) || ((uintptr_t)dev_out & 1))
    return fail(NZ_ERR_ALIGN, "misaligned indices or output");
  hipStream_t st = (hipStream_t)stream;
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  if (it == m->entries.end()) return fail(NZ_ERR_NOT_FOUND, "Data not found");
  if (int rc = refuse_under_capture(st, true, "gather_rows")) return rc;
  if (int rc = order_scratch_use(m, st)) return rc;
  if (int rc = settle_entry(m, it->second)) return rc;
  const Entry& ent = it->second;
  if (row_len == 0 || ent.n == 0 || ent.n % row_len)
    return fail(NZ_ERR_ARG, "stored tensor is not a table with rows of row_len elements");
  NzGeom g;
  if (int rc = make_geom(&g, ent.n, ent.chunk_syms, ent.lane_syms)) return rc;
  // chunks a row can touch: one when rows never straddle a chunk boundary, else
  // as many as a row can reach wherever it starts
  const uint32_t cpr = (row_len <= g.chunk_syms && g.chunk_syms % row_len == 0)
                           ? 1u
                           : (uint32_t)(((uint64_t)row_len + g.chunk_syms - 2) / g.chunk_syms + 1);
  // One chunk-sized slot per (row, touched chunk), taken from the encode scratch
  // of this manager.  The rows are served in slices, so that the slots of a
  // slice stay below a quarter GiB and its grid inside the launch limits,
  // whatever the number of rows; everything is validated before the first launch.
  const uint64_t slot_bytes = (uint64_t)cpr * g.chunk_syms * 2;
  const uint64_t cap_bytes = 256ull << 20;
  uint64_t per_slice = cap_bytes / slot_bytes;
  if (per_slice == 0) per_slice = 1;
  if (per_slice > count) per_slice = count;
  const uint32_t bx = (row_len + 255) / 256 < 64 ? (row_len + 255) / 256 : 64;
  if (per_slice * cpr > 0x7FFFFFFFull || per_slice * bx > 0x7FFFFFFFull)
    per_slice = 0x7FFFFFFFull / (cpr > bx ? cpr : bx);
  const uint64_t need = per_slice * slot_bytes;
  if (m->ws_bytes < need) {
    NZ_HIP(hipStreamSynchronize(st));
    if (int rc = settle_all(m)) return rc;
    if (m->ws) NZ_HIP(hipFree(m->ws));
    m->ws = nullptr;
    m->ws_bytes = 0;
    NZ_HIP(hipMalloc(&m->ws, need));
    m->ws_bytes = need;
  }
  const NzNorm nm{m->normalizer ? (const uint8_t*)ent.norm : nullptr, log2_of(m->normalizer ? m->normalizer : 1)};
  uint16_t* scratch = (uint16_t*)m->ws;
  for (uint64_t at = 0; at < count; at += per_slice) {
    const uint32_t rows_now = (uint32_t)(count - at < per_slice ? count - at : per_slice);
    const long long* idx = (const long long*)dev_indices + at;
#define NZ_ROWS_CASE(S)                                                                              \
  nz_launch_rows<S>(g, ent.comp, ent.comp_bytes, ent.packed, scratch, m->d_status, nm, idx,         \
                    rows_now, row_len, cpr, st)
    switch (m->precision) {
      case 7: NZ_ROWS_CASE(7); break;
      case 3: NZ_ROWS_CASE(3); break;
      case 1: NZ_ROWS_CASE(1); break;
      default: NZ_ROWS_CASE(0); break;
    }
#undef NZ_ROWS_CASE
    NZ_HIP(hipGetLastError());
    hipLaunchKernelGGL(nz_copy_rows_kernel, dim3(bx * rows_now), dim3(256), 0, st, (const uint16_t*)scratch, idx,
                       ent.n / row_len, row_len, g.chunk_syms, cpr, bx, (uint16_t*)dev_out + at * (uint64_t)row_len);
    NZ_HIP(hipGetLastError());
  }
  return NZ_OK;
}

int nz_manager_geometry(nz_manager* m, const char* name, uint32_t* chunk_size, uint32_t* lane_syms) {
  if (!m || !name) return fail(NZ_ERR_ARG, "null manager or name");
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  if (it == m->entries.end()) return fail(NZ_ERR_NOT_FOUND, "Data not found");
  if (chunk_size) *chunk_size = it->second.chunk_syms;
  if (lane_syms) *lane_syms = it->second.lane_syms;
  return NZ_OK;
}

int nz_manager_geometry_hint(nz_manager* m, const char* name, uint32_t chunk_size, uint32_t lane_syms) {
  if (!m || !name) return fail(NZ_ERR_ARG, "null manager or name");
  std::lock_guard<std::mutex> lock(m->mu);
  if (chunk_size == 0 && lane_syms == 0) {
    m->hints.erase(name);
    return NZ_OK;
  }
  if (nz_geom_check(chunk_size, lane_syms))
    return fail(NZ_ERR_ARG,
                "unsupported geometry: lane_syms must be a multiple of 8 (>= 16), chunk_size a multiple "
                "of 512 cut into 1..8 segments of 64*lane_syms, the last one at least 1024 long");
  m->hints[name] = std::make_pair(chunk_size, lane_syms);
  return NZ_OK;
}

int nz_manager_meta(nz_manager* m, const char* name, uint64_t* numel, int* dtype) {
  if (!m || !name) return fail(NZ_ERR_ARG, "null manager or name");
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  if (it == m->entries.end()) return fail(NZ_ERR_NOT_FOUND, "Data not found");
  if (numel) *numel = it->second.n;
  if (dtype) *dtype = it->second.dtype;
  return NZ_OK;
}

uint64_t nz_manager_size(nz_manager* m, const char* name) {
  if (!m || !name) return 0;
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  if (it == m->entries.end()) return 0;  // cuda/high_level.cu:209-211
  if (settle_entry(m, it->second)) return 0;  // the size is not known: nz_last_error() says why
  return it->second.comp_bytes + it->second.packed_bytes + it->second.norm_bytes;
}

uint64_t nz_manager_size_reference(nz_manager* m, const char* name) {
  if (!m || !name) return 0;
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  if (it == m->entries.end()) return 0;
  if (settle_entry(m, it->second)) return 0;
  const Entry& e = it->second;
  // cuda/high_level.cu:89-93: without normalizers the reference still allocates
  // (and size() counts, :208-221) one byte per 1024 elements
  const uint64_t idle_norm = m->normalizer ? 0 : (e.n + 1023) / 1024;
  return e.comp_bytes + e.packed_bytes + e.norm_bytes + idle_norm;
}

uint64_t nz_manager_exp_bytes(nz_manager* m, const char* name) {
  if (!m || !name) return 0;
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  if (it == m->entries.end()) return 0;
  if (settle_entry(m, it->second)) return 0;
  return it->second.comp_bytes;
}

uint64_t nz_manager_packed_bytes(nz_manager* m, const char* name) {
  if (!m || !name) return 0;
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  return it == m->entries.end() ? 0 : it->second.packed_bytes;
}

int nz_manager_buffers(nz_manager* m, const char* name, const void** dev_comp, uint64_t* comp_bytes,
                       const void** dev_packed, uint64_t* packed_bytes) {
  if (!m || !name) return fail(NZ_ERR_ARG, "null manager or name");
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  if (it == m->entries.end()) return fail(NZ_ERR_NOT_FOUND, "Data not found");
  if (int rc = settle_entry(m, it->second)) return rc;
  if (dev_comp) *dev_comp = it->second.comp;
  if (comp_bytes) *comp_bytes = it->second.comp_bytes;
  if (dev_packed) *dev_packed = it->second.packed;
  if (packed_bytes) *packed_bytes = it->second.packed_bytes;
  return NZ_OK;
}

uint64_t nz_manager_norm_bytes(nz_manager* m, const char* name) {
  if (!m || !name) return 0;
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  return it == m->entries.end() ? 0 : it->second.norm_bytes;
}

int nz_manager_export(nz_manager* m, const char* name, void* host_comp, uint64_t comp_cap,
                      void* host_packed, uint64_t packed_cap, void* host_norm, uint64_t norm_cap,
                      void* stream) {
  if (!m || !name) return fail(NZ_ERR_ARG, "null manager or name");
  hipStream_t st = (hipStream_t)stream;
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  if (it == m->entries.end()) return fail(NZ_ERR_NOT_FOUND, "Data not found");
  if (int rc = settle_entry(m, it->second)) return rc;
  const Entry& ent = it->second;
  if (comp_cap < ent.comp_bytes || packed_cap < ent.packed_bytes || norm_cap < ent.norm_bytes)
    return fail(NZ_ERR_CAPACITY, "host buffers smaller than the stored streams");
  if ((ent.comp_bytes && !host_comp) || (ent.packed_bytes && !host_packed) || (ent.norm_bytes && !host_norm))
    return fail(NZ_ERR_ARG, "null host buffer");
  if (ent.norm_bytes) NZ_HIP(hipMemcpyAsync(host_norm, ent.norm, ent.norm_bytes, hipMemcpyDeviceToHost, st));
  if (ent.comp_bytes) NZ_HIP(hipMemcpyAsync(host_comp, ent.comp, ent.comp_bytes, hipMemcpyDeviceToHost, st));
  if (ent.packed_bytes)
    NZ_HIP(hipMemcpyAsync(host_packed, ent.packed, ent.packed_bytes, hipMemcpyDeviceToHost, st));
  NZ_HIP(hipStreamSynchronize(st));
  return NZ_OK;
}

int nz_manager_import(nz_manager* m, const char* name, const void* host_comp, uint64_t comp_bytes,
                      const void* host_packed, uint64_t packed_bytes, const void* host_norm,
                      uint64_t norm_bytes, void* stream) {
  if (!m || !name || !host_comp) return fail(NZ_ERR_ARG, "null manager, name or container");
  hipStream_t st = (hipStream_t)stream;
  // the container describes itself: check it against this manager before anything is stored
  if (comp_bytes < NZ_HEADER_BYTES) return fail(NZ_ERR_CORRUPT, "container shorter than its header");
  uint32_t h[16];
  std::memcpy(h, host_comp, sizeof(h));
  if (h[0] != NZ_MAGIC) return fail(NZ_ERR_CORRUPT, "not an exponent container");
  if (h[1] != NZ_FORMAT_VERSION) return fail(NZ_ERR_CORRUPT, "container of another format version");
  const uint64_t n = (uint64_t)h[2] | ((uint64_t)h[3] << 32);
  const uint64_t total = (uint64_t)h[10] | ((uint64_t)h[11] << 32);
  std::lock_guard<std::mutex> lock(m->mu);
  NzGeom g;
  if (nz_geom_make(&g, n, h[4], h[5])) return fail(NZ_ERR_CORRUPT, "container header holds an unsupported geometry");
  if (h[6] != (uint32_t)g.n_chunks || h[7] != (uint32_t)g.n_segs || h[8] != g.dir_off || h[9] != g.rec_off ||
      total != comp_bytes || total > nz_geom_bound(&g) || total < g.rec_off + NZ_TAIL_PAD)
    return fail(NZ_ERR_CORRUPT, "container header is inconsistent");
  if (packed_bytes != nz_packed_stored_bytes_of(&g, m->precision))
    return fail(NZ_ERR_ARG, "packed stream does not have the size this manager's precision gives");
  if (packed_bytes && !host_packed) return fail(NZ_ERR_ARG, "null packed stream");
  if (norm_bytes != norm_bytes_of(n, m->normalizer))
    return fail(NZ_ERR_ARG, "normalizer bytes do not have the size this manager's normalizer_size gives");
  if (norm_bytes && !host_norm) return fail(NZ_ERR_ARG, "null normalizer bytes");
  // the directory must be non-decreasing and end where the container ends
  {
    const uint8_t* c = (const uint8_t*)host_comp;
    uint32_t prev = 0;
    for (uint64_t i = 0; i <= g.n_segs; ++i) {
      uint32_t v;
      std::memcpy(&v, c + g.dir_off + 4 * i, 4);
      if (v < prev) return fail(NZ_ERR_CORRUPT, "container directory is not monotone");
      prev = v;
    }
    if (g.rec_off + 4 * (uint64_t)prev + NZ_TAIL_PAD != total)
      return fail(NZ_ERR_CORRUPT, "container directory does not match its size");
  }
  Entry ent;
  ent.n = n;
  ent.dtype = NZ_DTYPE_BF16;
  ent.lane_syms = h[5];
  ent.chunk_syms = h[4];
  ent.comp_bytes = ent.comp_cap = comp_bytes;
  ent.packed_bytes = packed_bytes;
  ent.packed_cap = packed_bytes + 16;  // never a zero-byte allocation; the slack is zeroed
  ent.norm_bytes = norm_bytes;
  ent.norm_cap = norm_bytes ? norm_bytes + 8 : 0;
  hipError_t e = hipMalloc(&ent.comp, ent.comp_cap);
  if (e == hipSuccess) e = hipMalloc(&ent.packed, ent.packed_cap);
  if (e == hipSuccess && norm_bytes) e = hipMalloc(&ent.norm, ent.norm_cap);
  if (e == hipSuccess && norm_bytes)
    e = hipMemcpyAsync(ent.norm, host_norm, norm_bytes, hipMemcpyHostToDevice, st);
  if (e == hipSuccess) e = hipMemcpyAsync(ent.comp, host_comp, comp_bytes, hipMemcpyHostToDevice, st);
  if (e == hipSuccess && packed_bytes)
    e = hipMemcpyAsync(ent.packed, host_packed, packed_bytes, hipMemcpyHostToDevice, st);
  if (e == hipSuccess) e = hipMemsetAsync((uint8_t*)ent.packed + packed_bytes, 0, 16, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);  // the host buffers are the caller's again
  if (e != hipSuccess) {
    if (ent.comp) (void)hipFree(ent.comp);
    if (ent.packed) (void)hipFree(ent.packed);
    if (ent.norm) (void)hipFree(ent.norm);
    return fail(NZ_ERR_HIP, std::string("import: ") + hipGetErrorString(e));
  }
  auto it = m->entries.find(name);
  if (it != m->entries.end()) {
    // kernels reading the old buffers may still be in flight
    (void)hipDeviceSynchronize();
    // the outcome of a rewrite that was still pending no longer matters: the entry is replaced
    // whole (a slot that could not be settled skips entries that are gone)
    (void)settle_entry(m, it->second);
    release_entry(it->second);
    m->entries.erase(it);
  }
  m->entries.emplace(name, ent);
  return NZ_OK;
}

int nz_manager_erase(nz_manager* m, const char* name) {
  if (!m || !name) return fail(NZ_ERR_ARG, "null manager or name");
  std::lock_guard<std::mutex> lock(m->mu);
  auto it = m->entries.find(name);
  if (it == m->entries.end()) return fail(NZ_ERR_NOT_FOUND, "Data not found");
  // kernels reading these buffers may still be in flight
  NZ_HIP(hipDeviceSynchronize());
  if (int rc = settle_entry(m, it->second)) return rc;
  if (it->second.comp) (void)hipFree(it->second.comp);
  if (it->second.packed) (void)hipFree(it->second.packed);
  if (it->second.norm) (void)hipFree(it->second.norm);
  m->entries.erase(it);
  return NZ_OK;
}

int nz_manager_trim(nz_manager* m) {
  if (!m) return fail(NZ_ERR_ARG, "null manager");
  std::lock_guard<std::mutex> lock(m->mu);
  // kernels of earlier writes, gathers or products may still use the scratch
  NZ_HIP(hipDeviceSynchronize());
  if (int rc = settle_all(m)) return rc;
  if (m->ws) NZ_HIP(hipFree(m->ws));
  m->ws = nullptr;
  m->ws_bytes = 0;
  for (int k = 0; k < 2; ++k) {
    if (m->rw[k].ws) NZ_HIP(hipFree(m->rw[k].ws));
    m->rw[k].ws = nullptr;
    m->rw[k].ws_bytes = 0;
  }
  if (m->gemv_acc) NZ_HIP(hipFree(m->gemv_acc));
  m->gemv_acc = nullptr;
  m->gemv_rows = 0;
  return NZ_OK;
}

int nz_manager_rewrite_stats(nz_manager* m, uint64_t* in_place_batches, uint64_t* outgrown_entries,
                             uint64_t* placed_again) {
  if (!m) return fail(NZ_ERR_ARG, "null manager");
  std::lock_guard<std::mutex> lock(m->mu);
  if (int rc = settle_all(m)) return rc;
  if (in_place_batches) *in_place_batches = m->rewrites;
  if (outgrown_entries) *outgrown_entries = m->rewrites_replaced;
  if (placed_again) *placed_again = m->rewrites_redone;
  return NZ_OK;
}

int nz_manager_check(nz_manager* m, void* stream) {
  if (!m) return fail(NZ_ERR_ARG, "null manager");
  hipStream_t st = (hipStream_t)stream;
  std::lock_guard<std::mutex> lock(m->mu);
  m->h_pin[16] = 0;
  NZ_HIP(hipMemcpyAsync(&m->h_pin[16], m->d_status, 4, hipMemcpyDeviceToHost, st));
  NZ_HIP(hipMemsetAsync(m->d_status, 0, 4, st));
  NZ_HIP(hipStreamSynchronize(st));
  const uint32_t hs = (uint32_t)m->h_pin[16];
  // a product that met a broken container left rows half summed: start clean
  if (hs && m->gemv_acc) NZ_HIP(hipMemset(m->gemv_acc, 0, m->gemv_rows * 16));
  if (hs == 8u) return fail(NZ_ERR_CORRUPT, "a row gather was given an index outside the table");
  if (hs)
    return fail(NZ_ERR_CORRUPT,
                "a read saw a container that failed validation (status " + std::to_string(hs) + ")");
  return NZ_OK;
}

}  // extern "C"
