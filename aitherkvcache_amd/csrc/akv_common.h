// Shared device/host helpers for the gfx950 TurboQuant kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/aitherkv.h"

#define AKV_WAVE 64

// ----------------------------------------------------------------------------------
// host: status + message
// ----------------------------------------------------------------------------------
char* akv_error_buffer();  // thread-local, 512 bytes (defined in akv_codec.hip)

static inline int akv_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(akv_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

#define AKV_REQUIRE(cond, ...)                                  \
  do {                                                          \
    if (!(cond)) return akv_fail(AKV_ERR_INVALID, __VA_ARGS__); \
  } while (0)

#define AKV_HIP(call)                                                                         \
  do {                                                                                        \
    hipError_t e_ = (call);                                                                   \
    if (e_ != hipSuccess)                                                                     \
      return akv_fail(AKV_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_),     \
                      __FILE__, __LINE__);                                                    \
  } while (0)

#define AKV_LAUNCH_CHECK(name)                                                                \
  do {                                                                                        \
    hipError_t e_ = hipGetLastError();                                                        \
    if (e_ != hipSuccess)                                                                     \
      return akv_fail(AKV_ERR_HIP, "launch of %s failed: %s", name, hipGetErrorString(e_));   \
  } while (0)

static inline bool akv_valid_dtype(int t) { return t == AKV_F16 || t == AKV_BF16 || t == AKV_F32; }
static inline bool akv_valid_itype(int t) { return t == AKV_I32 || t == AKV_I64; }
static inline int akv_packed_size(int d, int bits) { return d * bits / 8; }

int akv_cached_cu_count();  // 0 when no device (defined in akv_codec.hip)

// Timing of the dominant kernel of an entry point (akv_profile_enable).  AKV_LAUNCH_TIMED attaches the
// `end` event of the next ring pair to the kernel's own dispatch and the `begin` event to the dispatch of
// a one-thread stamp kernel launched right before it: the elapsed time between the two is the kernel's
// duration from the end of the preceding dispatch, which is what a kernel trace of back-to-back launches
// reports.  (Events recorded around the launch put barrier packets next to it, and the time the command
// processor spends on those -- about 5 us -- lands inside the measurement.)  mark_begin / mark_end are
// that bracketing form, kept for the kernels that are nobody's headline.
void akv_profile_mark_begin(hipStream_t s);
void akv_profile_mark_end(hipStream_t s);
bool akv_profile_take(hipEvent_t* begin, hipEvent_t* end);
void akv_profile_stamp(hipStream_t s, hipEvent_t begin);
#define AKV_LAUNCH_TIMED(kern, grid, block, lds, stream, ...)                                                  \
  do {                                                                                                         \
    hipEvent_t akv_b_, akv_e_;                                                                                 \
    if (akv_profile_take(&akv_b_, &akv_e_)) {                                                                  \
      akv_profile_stamp(stream, akv_b_);                                                                       \
      hipExtLaunchKernelGGL(kern, dim3(grid), dim3(block), (uint32_t)(lds), stream, nullptr, akv_e_, 0, __VA_ARGS__); \
    } else {                                                                                                   \
      hipLaunchKernelGGL(kern, dim3(grid), dim3(block), (uint32_t)(lds), stream, __VA_ARGS__);                 \
    }                                                                                                          \
  } while (0)

// Offsets (in floats) into the prepared-rotation buffer.
//   [0, d*d)        Pi     row-major  (y_i = sum_j Pi[i][j] x_j)
//   [d*d, 2*d*d)    Pi^T   row-major
//   [2*d*d, ...)    d = 128 only: float16 hi/lo operand tiles of the MFMA encode kernel (64 KB),
//                   a flag word (256 B reserved), the same for the MFMA decode kernel (64 KB)
static inline size_t akv_prep_floats(int d) { return (size_t)4 * d * d + 1024; }
#define AKV_PREP_DECODE_OFFSET(d) ((size_t)2 * (d) * (d) * 4 + 65536 + 256)

// Arguments of the encode / decode kernels (flat and paged forms share one struct).
struct akv_gen_args {
  // encode input
  const void* x;
  int64_t n;        // vectors (paged: num_tokens * num_kv_heads)
  int64_t xs0, xs1; // flat: xs0 = row stride; paged: xs0 = token stride, xs1 = head stride
  int heads;        // paged: num_kv_heads
  const void* slots;
  int slot_itype;
  int block_size;
  int64_t max_blocks;
  const float* mat;   // [D][D] staged matrix, [k][out]
  const float* table; // boundaries (encode) or centroids (decode)
  // packed side
  uint8_t* packed;
  int64_t ps0, ps1, ps2; // flat: ps0 = row stride (bytes); paged: blk, pos, head strides (bytes)
  float* norms;
  int64_t ns0, ns1, ns2;
  // paged encode of a second tensor in the same launch (K and V of one step): same shapes, strides and
  // slots as x / packed / norms; vectors n .. 2n - 1 of the launch.  Null when there is none.
  const void* x2;
  uint8_t* packed2;
  float* norms2;
  // decode output
  void* out;
  int64_t os0, os1, os2;  // flat: os0 = row stride; block-wise decode: blk, pos, head strides (elements)
};

// ----------------------------------------------------------------------------------
// device: element loads / stores
// ----------------------------------------------------------------------------------
struct akv_f16 { uint16_t v; };
struct akv_bf16 { uint16_t v; };

__device__ __forceinline__ float akv_to_float(__half h) { return __half2float(h); }
__device__ __forceinline__ float akv_bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
__device__ __forceinline__ uint16_t akv_float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);                                            // RNE
  return (uint16_t)(u >> 16);
}

template <int DT> struct akv_elem;
template <> struct akv_elem<AKV_F16> {
  typedef __half type;
  static __device__ __forceinline__ float load(const void* p, int64_t i) {
    return __half2float(((const __half*)p)[i]);
  }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) {
    ((__half*)p)[i] = __float2half_rn(v);
  }
};
template <> struct akv_elem<AKV_BF16> {
  typedef uint16_t type;
  static __device__ __forceinline__ float load(const void* p, int64_t i) {
    return akv_bf16_bits_to_float(((const uint16_t*)p)[i]);
  }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) {
    ((uint16_t*)p)[i] = akv_float_to_bf16_bits(v);
  }
};
template <> struct akv_elem<AKV_F32> {
  typedef float type;
  static __device__ __forceinline__ float load(const void* p, int64_t i) {
    return ((const float*)p)[i];
  }
  static __device__ __forceinline__ void store(void* p, int64_t i, float v) {
    ((float*)p)[i] = v;
  }
};

__device__ __forceinline__ int64_t akv_load_index(const void* p, int itype, int64_t i) {
  return itype == AKV_I64 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}

// ----------------------------------------------------------------------------------
// device: float32 operations that stay rounded one by one.  (The "_rn" helpers of the HIP headers are
// plain operators, which the compiler is free to fuse into multiply-adds; a product made here carries
// no permission to be fused, so a sum that takes it sees the rounded product, as in code that runs
// one tensor operation after the other.)
// ----------------------------------------------------------------------------------
__device__ __forceinline__ float akv_mul_rn(float a, float b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float akv_add_rn(float a, float b) {
#pragma clang fp contract(off)
  return a + b;
}
__device__ __forceinline__ float akv_sub_rn(float a, float b) {
#pragma clang fp contract(off)
  return a - b;
}

// ----------------------------------------------------------------------------------
// device: the value of lane (lane ^ M), by data-parallel primitives and the row swaps: no trip through the LDS
// crossbar (a shuffle is one, some hundred cycles under load).  M is a power of two below 64.
// ----------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ uint32_t akv_dpp_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}
template <int M>
__device__ __forceinline__ uint32_t akv_lane_xor_u32(uint32_t v) {
  static_assert(M == 1 || M == 2 || M == 4 || M == 8 || M == 16 || M == 32, "a single bit of the lane number");
  if constexpr (M == 1) return akv_dpp_u32<0xB1>(v);                      // quad_perm [1,0,3,2]
  else if constexpr (M == 2) return akv_dpp_u32<0x4E>(v);                 // quad_perm [2,3,0,1]
  else if constexpr (M == 4) return akv_dpp_u32<0x141>(akv_dpp_u32<0x1B>(v));   // quad_perm [3,2,1,0] (^3), then row_half_mirror (^7)
  else if constexpr (M == 8) return akv_dpp_u32<0x128>(v);                // row_ror:8
  else {
    // fed the same value twice, the swaps leave (rows 0,1,0,1 | 2,3,2,3) and (rows 0,0,2,2 | 1,1,3,3)
    const bool upper = (threadIdx.x & M) != 0;
    if constexpr (M == 16) {
      auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
      return upper ? r[0] : r[1];
    } else {
      auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
      return upper ? r[0] : r[1];
    }
  }
}
template <int M> __device__ __forceinline__ float akv_lane_xor(float v) {
  return __uint_as_float(akv_lane_xor_u32<M>(__float_as_uint(v)));
}
template <int M> __device__ __forceinline__ int akv_lane_xor(int v) { return (int)akv_lane_xor_u32<M>((uint32_t)v); }

// ----------------------------------------------------------------------------------
// device: wavefront (64-lane) reductions; every lane receives the result.  (The butterfly of a shuffle loop
// -- partner lane ^ 32 first, lane ^ 1 last -- so the sums round as they always did.)
// ----------------------------------------------------------------------------------
__device__ __forceinline__ float akv_wave_sum(float v) {
  v += akv_lane_xor<32>(v);
  v += akv_lane_xor<16>(v);
  v += akv_lane_xor<8>(v);
  v += akv_lane_xor<4>(v);
  v += akv_lane_xor<2>(v);
  v += akv_lane_xor<1>(v);
  return v;
}
__device__ __forceinline__ float akv_wave_max(float v) {
  v = fmaxf(v, akv_lane_xor<32>(v));
  v = fmaxf(v, akv_lane_xor<16>(v));
  v = fmaxf(v, akv_lane_xor<8>(v));
  v = fmaxf(v, akv_lane_xor<4>(v));
  v = fmaxf(v, akv_lane_xor<2>(v));
  v = fmaxf(v, akv_lane_xor<1>(v));
  return v;
}
__device__ __forceinline__ int akv_wave_sum(int v) {
  v += akv_lane_xor<32>(v);
  v += akv_lane_xor<16>(v);
  v += akv_lane_xor<8>(v);
  v += akv_lane_xor<4>(v);
  v += akv_lane_xor<2>(v);
  v += akv_lane_xor<1>(v);
  return v;
}
// inclusive prefix sum over the 64 lanes: shifts inside the rows of sixteen (lanes without a source add zero),
// then the totals of the rows below
__device__ __forceinline__ int akv_wave_inclusive_scan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111 /*row_shr:1*/, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x112 /*row_shr:2*/, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x114 /*row_shr:4*/, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x118 /*row_shr:8*/, 0xf, 0xf, true);
  const int t0 = __builtin_amdgcn_readlane(v, 15), t1 = __builtin_amdgcn_readlane(v, 31), t2 = __builtin_amdgcn_readlane(v, 47);
  const int row = (threadIdx.x & 63) >> 4;
  return v + (row >= 1 ? t0 : 0) + (row >= 2 ? t1 : 0) + (row >= 3 ? t2 : 0);
}

// ----------------------------------------------------------------------------------
// device: MSB-first code streams (covers pack_4bit / pack_2bit / pack_3bit of
// aither_kvcache/packing.py and pack_multibit of hybrid_quantizer.py:310-352 -- all four
// are the same big-endian bit stream with BITS bits per index)
// ----------------------------------------------------------------------------------
// Byte k of the stream, given a callable code_of(dim).
template <int BITS, class F>
__device__ __forceinline__ uint32_t akv_stream_byte(int k, F code_of) {
  const int p0 = 8 * k;
  const int dim0 = p0 / BITS;
  const int dim1 = (p0 + 7) / BITS;
  uint32_t byte = 0;
  for (int dim = dim0; dim <= dim1; ++dim) {
    const uint32_t c = code_of(dim);
    const int shift = (p0 + 8) - (dim * BITS + BITS);
    byte |= shift >= 0 ? (c << shift) : (c >> (-shift));
  }
  return byte & 0xffu;
}

// Index `dim` of the stream, given a callable byte_of(offset).
template <int BITS, class F>
__device__ __forceinline__ uint32_t akv_stream_code(int dim, F byte_of) {
  const int p = dim * BITS;
  const int o = p >> 3;
  const int r = p & 7;
  uint32_t w = byte_of(o) << 8;
  if (r + BITS > 8) w |= byte_of(o + 1);
  return (w >> (16 - BITS - r)) & ((1u << BITS) - 1u);
}

// code = #{b in boundaries : b < y}  (torch.searchsorted(right=False), quantizer.py:203-207)
template <int BITS>
__device__ __forceinline__ uint32_t akv_search(float y, const float* bnd) {
  uint32_t c = 0;
#pragma unroll
  for (int k = 0; k < (1 << BITS) - 1; ++k) c += (bnd[k] < y) ? 1u : 0u;
  if (y != y) c = (1u << BITS) - 1u;  // searchsorted places NaN after every boundary
  return c;
}
