// Host-side launchers of the kernels that exist once per precision (kept
// mantissa bits S = 7, 3, 1, 0).  nz_launch.hip is compiled once per precision
// (-DNZ_S=...) and defines them for that S; nz_api.hip only declares them, so
// that the precisions compile side by side.
#pragma once

#include <hip/hip_runtime.h>

#include "nz_kernels.hip"

// Allow the register encode kernels of precision S up to 96 KiB of dynamic LDS
// (more than 64 KiB has to be asked for once per kernel and device).
template <int S>
hipError_t nz_allow_encode_lds();

// cls 0..3: nz_encode_kernel<S, 8 | 16 | 32 | 36> (segments of up to 64 / 128 / 256 /
// 288 symbols per lane, coded from registers); 4: nz_encode_long_kernel<S>
template <int S>
void nz_launch_encode(const NzEncBatch& b, int cls, dim3 grid, dim3 block, uint32_t lds, hipStream_t st);

template <int S>
void nz_launch_decode(const NzGeom& g, const void* comp, uint64_t comp_bytes, const void* packed, void* out,
                      uint32_t* d_status, const NzNorm& nm, uint32_t stream_out, hipStream_t st);

template <int S>
void nz_launch_decode_batch(const NzBatch& b, uint32_t grid, uint32_t max_spc, bool stream_out, uint32_t* d_status,
                            hipStream_t st);

template <int S>
void nz_launch_gemv(const NzBatch& b, uint32_t grid, uint32_t max_spc, uint32_t* d_status, hipStream_t st);

template <int S>
void nz_launch_rows(const NzGeom& g, const void* comp, uint64_t comp_bytes, const void* packed, uint16_t* scratch,
                    uint32_t* d_status, const NzNorm& nm, const long long* idx, uint32_t count, uint32_t row_len,
                    uint32_t cpr, hipStream_t st);

#ifndef NZ_S
#define NZ_DECLARE_PRECISION(S)                                                                                      \
  extern template hipError_t nz_allow_encode_lds<S>();                                                               \
  extern template void nz_launch_encode<S>(const NzEncBatch&, int, dim3, dim3, uint32_t, hipStream_t);               \
  extern template void nz_launch_decode<S>(const NzGeom&, const void*, uint64_t, const void*, void*, uint32_t*,      \
                                           const NzNorm&, uint32_t, hipStream_t);                                    \
  extern template void nz_launch_decode_batch<S>(const NzBatch&, uint32_t, uint32_t, bool, uint32_t*, hipStream_t);  \
  extern template void nz_launch_gemv<S>(const NzBatch&, uint32_t, uint32_t, uint32_t*, hipStream_t);                \
  extern template void nz_launch_rows<S>(const NzGeom&, const void*, uint64_t, const void*, uint16_t*, uint32_t*,    \
                                         const NzNorm&, const long long*, uint32_t, uint32_t, uint32_t, hipStream_t);
NZ_DECLARE_PRECISION(7)
NZ_DECLARE_PRECISION(3)
NZ_DECLARE_PRECISION(1)
NZ_DECLARE_PRECISION(0)
#undef NZ_DECLARE_PRECISION
#endif
