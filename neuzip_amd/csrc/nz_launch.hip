// The kernels of ONE precision (compile with -DNZ_S=7, 3, 1 or 0) and their
// host-side launchers; see nz_launch.h.
#ifndef NZ_S
#error "compile with -DNZ_S=<kept mantissa bits>"
#endif
#define NZ_TEMPLATES_ONLY
#include "nz_launch.h"

template <int S>
hipError_t nz_allow_encode_lds() {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&nz_encode_kernel<S, 8>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
  if (e == hipSuccess)
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&nz_encode_kernel<S, 16>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
  if (e == hipSuccess)
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&nz_encode_kernel<S, 32>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
  if (e == hipSuccess)
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&nz_encode_kernel<S, 36>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
  return e;
}

template <int S>
void nz_launch_encode(const NzEncBatch& b, int cls, dim3 grid, dim3 block, uint32_t lds, hipStream_t st) {
  switch (cls) {
    case 0: hipLaunchKernelGGL((nz_encode_kernel<S, 8>), grid, block, lds, st, b); break;
    case 1: hipLaunchKernelGGL((nz_encode_kernel<S, 16>), grid, block, lds, st, b); break;
    case 2: hipLaunchKernelGGL((nz_encode_kernel<S, 32>), grid, block, lds, st, b); break;
    case 3: hipLaunchKernelGGL((nz_encode_kernel<S, 36>), grid, block, lds, st, b); break;
    default: hipLaunchKernelGGL((nz_encode_long_kernel<S>), grid, dim3(NZ_ENC_LONG_THREADS), 0, st, b); break;
  }
}

template <int S>
void nz_launch_decode(const NzGeom& g, const void* comp, uint64_t comp_bytes, const void* packed, void* out,
                      uint32_t* d_status, const NzNorm& nm, uint32_t stream_out, hipStream_t st) {
  const size_t lds = NZ_DEC_LDS_BYTES(g.spc);
  const dim3 gd((uint32_t)g.n_chunks), bd(64 * g.spc);
#define NZ_DEC_LAUNCH(NORM, STREAM)                                                                            \
  hipLaunchKernelGGL((nz_decode_kernel<S, NORM, STREAM>), gd, bd, lds, st, (const uint8_t*)comp, comp_bytes, \
                     (const uint8_t*)packed, (uint16_t*)out, g, d_status, nm)
  if (nm.bytes) {
    if (stream_out) NZ_DEC_LAUNCH(true, true);
    else NZ_DEC_LAUNCH(true, false);
  } else {
    if (stream_out) NZ_DEC_LAUNCH(false, true);
    else NZ_DEC_LAUNCH(false, false);
  }
#undef NZ_DEC_LAUNCH
}

template <int S>
void nz_launch_decode_batch(const NzBatch& b, uint32_t grid, uint32_t max_spc, bool stream_out, uint32_t* d_status,
                            hipStream_t st) {
  const size_t lds = NZ_DEC_LDS_BYTES(max_spc);
  const dim3 gd(grid), bd(64 * max_spc);
#define NZ_BATCH_LAUNCH(NORM, STREAM) \
  hipLaunchKernelGGL((nz_decode_batch_kernel<S, NORM, STREAM>), gd, bd, lds, st, b, d_status)
  if (b.item[0].norm) {
    if (stream_out) NZ_BATCH_LAUNCH(true, true);
    else NZ_BATCH_LAUNCH(true, false);
  } else {
    if (stream_out) NZ_BATCH_LAUNCH(false, true);
    else NZ_BATCH_LAUNCH(false, false);
  }
#undef NZ_BATCH_LAUNCH
}

template <int S>
void nz_launch_gemv(const NzBatch& b, uint32_t grid, uint32_t max_spc, uint32_t* d_status, hipStream_t st) {
  const size_t lds = NZ_DEC_LDS_BYTES(max_spc);
  const dim3 gd(grid), bd(64 * max_spc);
  // one activation row, or kernels that hold 2, 4 or 8 of them per lane (tensors with
  // normalizers: one row only, the caller has checked)
  if (b.item[0].norm) hipLaunchKernelGGL((nz_decode_gemv_kernel<S, true, 1>), gd, bd, lds, st, b, d_status);
  else if (b.x_rows <= 1) hipLaunchKernelGGL((nz_decode_gemv_kernel<S, false, 1>), gd, bd, lds, st, b, d_status);
  else if (b.x_rows <= 2) hipLaunchKernelGGL((nz_decode_gemv_kernel<S, false, 2>), gd, bd, lds, st, b, d_status);
  else if (b.x_rows <= 4) hipLaunchKernelGGL((nz_decode_gemv_kernel<S, false, 4>), gd, bd, lds, st, b, d_status);
  else hipLaunchKernelGGL((nz_decode_gemv_kernel<S, false, 8>), gd, bd, lds, st, b, d_status);
}

template <int S>
void nz_launch_rows(const NzGeom& g, const void* comp, uint64_t comp_bytes, const void* packed, uint16_t* scratch,
                    uint32_t* d_status, const NzNorm& nm, const long long* idx, uint32_t count, uint32_t row_len,
                    uint32_t cpr, hipStream_t st) {
  const size_t lds = NZ_DEC_LDS_BYTES(g.spc);
  const dim3 gd(count * cpr), bd(64 * g.spc);
  if (nm.bytes)
    hipLaunchKernelGGL((nz_decode_rows_kernel<S, true>), gd, bd, lds, st, (const uint8_t*)comp, comp_bytes,
                       (const uint8_t*)packed, scratch, g, d_status, nm, idx, row_len, cpr);
  else
    hipLaunchKernelGGL((nz_decode_rows_kernel<S, false>), gd, bd, lds, st, (const uint8_t*)comp, comp_bytes,
                       (const uint8_t*)packed, scratch, g, d_status, nm, idx, row_len, cpr);
}

// NZ_PART (optional) cuts the unit into parts that a build can compile side by side:
// 0 = the encode kernels, 1 = decode, batch decode and row gather, 2 = the fused products,
// 12 = both of the latter; undefined = everything.  (Every part parses all of the kernels'
// source again: on eight cores two parts per precision build fastest, 68 s against 80 s
// with three and 91 s with one.)
#if !defined(NZ_PART) || NZ_PART == 0
template hipError_t nz_allow_encode_lds<NZ_S>();
template void nz_launch_encode<NZ_S>(const NzEncBatch&, int, dim3, dim3, uint32_t, hipStream_t);
#endif
#if !defined(NZ_PART) || NZ_PART == 1 || NZ_PART == 12
template void nz_launch_decode<NZ_S>(const NzGeom&, const void*, uint64_t, const void*, void*, uint32_t*, const NzNorm&,
                                     uint32_t, hipStream_t);
template void nz_launch_decode_batch<NZ_S>(const NzBatch&, uint32_t, uint32_t, bool, uint32_t*, hipStream_t);
#endif
#if !defined(NZ_PART) || NZ_PART == 2 || NZ_PART == 12
template void nz_launch_gemv<NZ_S>(const NzBatch&, uint32_t, uint32_t, uint32_t*, hipStream_t);
#endif
#if !defined(NZ_PART) || NZ_PART == 1 || NZ_PART == 12
template void nz_launch_rows<NZ_S>(const NzGeom&, const void*, uint64_t, const void*, uint16_t*, uint32_t*,
                                   const NzNorm&, const long long*, uint32_t, uint32_t, uint32_t, hipStream_t);
#endif

#if defined(NZ_PROBE_PHASES) && NZ_S == 7 && (!defined(NZ_PART) || NZ_PART == 0)
// measurement build only: cycles spent per phase of nz_encode_kernel<7, *>, summed over workgroups
extern "C" int nz_probe_read(unsigned long long* out, int reset) {
  if (hipMemcpyFromSymbol(out, HIP_SYMBOL(nz_probe_acc), sizeof(unsigned long long) * 8) != hipSuccess) return 1;
  if (reset) {
    unsigned long long z[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (hipMemcpyToSymbol(HIP_SYMBOL(nz_probe_acc), z, sizeof(z)) != hipSuccess) return 1;
  }
  return 0;
}
#endif
