// TurboQuant codec kernels: rotation preparation, quantize+pack, unpack+lookup, encode
// (flat and paged scatter), decode.  General kernels (any float dtype, head_dim 64/128/256,
// 2/3/4-bit); the MFMA fast path for fp16 / head_dim 128 lives in akv_encode_mfma.hip.
#include "akv_common.h"

// ----------------------------------------------------------------------------------
// host state
// ----------------------------------------------------------------------------------
char* akv_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int akv_cached_cu_count() {
  static int cached = -1;
  if (cached < 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      cached = prop.multiProcessorCount;
    else
      return 0;
  }
  return cached;
}

// Ring of event pairs: nothing is read back between launches, so sampled calls run back to back
// like unsampled ones.  Once the ring is full, later pairs overwrite the oldest.
static constexpr int kProfRing = 64;
static bool g_profile_on = false;
static hipEvent_t g_ev_begin[kProfRing], g_ev_end[kProfRing];
static bool g_ev_created = false;
static long g_ev_count = 0;       // pairs recorded since akv_profile_enable(1)
static bool g_ev_open = false;    // a begin without its end

void akv_profile_mark_begin(hipStream_t s) {
  if (!g_profile_on) return;
  (void)hipEventRecord(g_ev_begin[g_ev_count % kProfRing], s);
  g_ev_open = true;
}
void akv_profile_mark_end(hipStream_t s) {
  if (!g_profile_on || !g_ev_open) return;
  (void)hipEventRecord(g_ev_end[g_ev_count % kProfRing], s);
  g_ev_open = false;
  ++g_ev_count;
}

bool akv_profile_take(hipEvent_t* begin, hipEvent_t* end) {
  if (!g_profile_on) return false;
  *begin = g_ev_begin[g_ev_count % kProfRing];
  *end = g_ev_end[g_ev_count % kProfRing];
  g_ev_open = false;
  ++g_ev_count;
  return true;
}

__global__ void akv_stamp_kernel() {}
void akv_profile_stamp(hipStream_t s, hipEvent_t begin) {
  hipExtLaunchKernelGGL(akv_stamp_kernel, dim3(1), dim3(1), 0, s, nullptr, begin, 0);
}

extern "C" int akv_profile_enable(int on) {
  if (on && !g_ev_created) {
    for (int i = 0; i < kProfRing; ++i) {
      AKV_HIP(hipEventCreate(&g_ev_begin[i]));
      AKV_HIP(hipEventCreate(&g_ev_end[i]));
    }
    g_ev_created = true;
  }
  g_profile_on = on != 0;
  if (on) { g_ev_count = 0; g_ev_open = false; }
  return AKV_OK;
}

extern "C" int akv_profile_last_ms(float* ms) {
  AKV_REQUIRE(ms != nullptr, "akv_profile_last_ms: null output");
  if (g_ev_count == 0) return akv_fail(AKV_ERR_INVALID, "akv_profile_last_ms: nothing recorded");
  const int i = (int)((g_ev_count - 1) % kProfRing);
  AKV_HIP(hipEventSynchronize(g_ev_end[i]));
  AKV_HIP(hipEventElapsedTime(ms, g_ev_begin[i], g_ev_end[i]));
  return AKV_OK;
}

extern "C" int akv_profile_mean_ms(float* ms, int* samples) {
  AKV_REQUIRE(ms != nullptr, "akv_profile_mean_ms: null output");
  if (g_ev_count == 0) return akv_fail(AKV_ERR_INVALID, "akv_profile_mean_ms: nothing recorded");
  const int n = (int)(g_ev_count < kProfRing ? g_ev_count : kProfRing);
  AKV_HIP(hipEventSynchronize(g_ev_end[(g_ev_count - 1) % kProfRing]));
  double acc = 0.0;
  for (int k = 0; k < n; ++k) {
    const int i = (int)((g_ev_count - 1 - k) % kProfRing);
    float t = 0.f;
    AKV_HIP(hipEventElapsedTime(&t, g_ev_begin[i], g_ev_end[i]));
    acc += t;
  }
  *ms = (float)(acc / n);
  if (samples) *samples = n;
  return AKV_OK;
}

extern "C" const char* akv_version(void) { return "aitherkv-hip 0.1 (gfx950)"; }
extern "C" const char* akv_last_error(void) { return akv_error_buffer(); }
extern "C" int akv_device_cu_count(int* cu_count) {
  AKV_REQUIRE(cu_count != nullptr, "akv_device_cu_count: null output");
  *cu_count = akv_cached_cu_count();
  if (*cu_count <= 0) return akv_fail(AKV_ERR_HIP, "no HIP device available");
  return AKV_OK;
}

// ----------------------------------------------------------------------------------
// rotation preparation
// ----------------------------------------------------------------------------------
__global__ void akv_prepare_rotation_kernel(const float* __restrict__ R, float* __restrict__ prep,
                                            int d) {
  // 32x32 tiled transpose through LDS; also copies Pi itself.
  __shared__ float tile[32][33];
  const int bx = blockIdx.x * 32, by = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 256 threads: ty 0..7
  for (int r = ty; r < 32; r += 8) {
    const float v = R[(size_t)(by + r) * d + bx + tx];
    prep[(size_t)(by + r) * d + bx + tx] = v;
    tile[r][tx] = v;
  }
  __syncthreads();
  float* RT = prep + (size_t)d * d;
  for (int r = ty; r < 32; r += 8) RT[(size_t)(bx + r) * d + by + tx] = tile[tx][r];
}

int akv_prepare_rotation_mfma(const float* rotation, int d, void* prep, hipStream_t stream);
int akv_prepare_decode_mfma(const float* rotation, int d, void* prep, hipStream_t stream);
int akv_decode_mfma_try(const akv_gen_args& a, bool blocks, int d, int bits, int out_dtype, const void* rot_prep,
                        hipStream_t stream);

extern "C" size_t akv_rotation_prepared_bytes(int d) { return akv_prep_floats(d) * sizeof(float); }

extern "C" int akv_rotation_prepare(const float* rotation, int d, void* prep, size_t prep_bytes,
                                    void* stream) {
  AKV_REQUIRE(rotation && prep, "akv_rotation_prepare: null pointer");
  AKV_REQUIRE(d == 64 || d == 128 || d == 256 || d == 512, "akv_rotation_prepare: head_dim %d not in {64,128,256,512}", d);
  AKV_REQUIRE(prep_bytes >= akv_rotation_prepared_bytes(d), "akv_rotation_prepare: prep buffer too small");
  AKV_REQUIRE(((uintptr_t)prep & 255) == 0, "akv_rotation_prepare: prep must be 256-byte aligned");
  dim3 grid(d / 32, d / 32);
  akv_prepare_rotation_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(rotation, (float*)prep, d);
  AKV_LAUNCH_CHECK("akv_prepare_rotation_kernel");
  if (d == 128) {
    int rc = akv_prepare_rotation_mfma(rotation, d, prep, (hipStream_t)stream);
    if (rc) return rc;
    return akv_prepare_decode_mfma(rotation, d, prep, (hipStream_t)stream);
  }
  return AKV_OK;
}

// ----------------------------------------------------------------------------------
// Read probe: what a kernel that does nothing but read reaches on this device.  Every lane sums 16-byte loads
// of a contiguous buffer (a wavefront covers 1 KB per instruction, four loads in flight per lane) and one value
// per workgroup is written so that the loads stay.  Timed like the dominant kernels (akv_profile_*).
// ----------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void akv_read_probe_kernel(const uint4* __restrict__ src, size_t n16, uint32_t* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  uint32_t acc = 0;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    acc += (a.x ^ a.y) + (a.z ^ a.w) + (b.x ^ b.y) + (b.z ^ b.w) + (c.x ^ c.y) + (c.z ^ c.w) + (d.x ^ d.y) + (d.z ^ d.w);
  }
  for (; i < n16; i += stride) {
    const uint4 a = src[i];
    acc += (a.x ^ a.y) + (a.z ^ a.w);
  }
  acc = (uint32_t)akv_wave_sum((float)(acc & 0xffffu));
  if ((threadIdx.x & 63) == 0) atomicAdd(&sink[blockIdx.x & 63], acc);
}

extern "C" int akv_debug_read_probe(const void* src, size_t bytes, void* sink256, void* stream_) {
  AKV_REQUIRE(src && sink256, "akv_debug_read_probe: null pointer");
  AKV_REQUIRE(((uintptr_t)src & 15) == 0 && bytes >= 16, "akv_debug_read_probe: src must be 16-byte aligned and hold 16 bytes or more");
  hipStream_t stream = (hipStream_t)stream_;
  const int cus = akv_cached_cu_count();
  const int grid = 2 * (cus > 0 ? cus : 256);     // measured best on the MI355X: 6.1 TB/s over 360 MB (1, 3, 4, 8, 16 per CU: 6.0, 5.8, 5.0, 4.8, 3.7)
  AKV_LAUNCH_TIMED(akv_read_probe_kernel, grid, 256, 0, stream, (const uint4*)src, bytes / 16, (uint32_t*)sink256);
  AKV_LAUNCH_CHECK("akv_read_probe_kernel");
  return AKV_OK;
}

// ----------------------------------------------------------------------------------
// quantize + pack / unpack + lookup   (triton_ops.py:220-259)
// ----------------------------------------------------------------------------------
template <int BITS>
__global__ __launch_bounds__(256) void akv_quantize_pack_kernel(
    const float* __restrict__ y, int64_t n, int d, int64_t y_stride,
    const float* __restrict__ bnd_g, uint8_t* __restrict__ out, int64_t out_stride) {
  __shared__ float bnd[16];
  if (threadIdx.x < (1 << BITS) - 1) bnd[threadIdx.x] = bnd_g[threadIdx.x];
  __syncthreads();
  const int P = d * BITS / 8;
  const int64_t total = n * P;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = i / P;
    const int k = (int)(i - row * P);
    const float* yr = y + row * y_stride;
    out[row * out_stride + k] =
        (uint8_t)akv_stream_byte<BITS>(k, [&](int dim) { return akv_search<BITS>(yr[dim], bnd); });
  }
}

template <int BITS>
__global__ __launch_bounds__(256) void akv_unpack_lookup_kernel(
    const uint8_t* __restrict__ packed, int64_t n, int d, int64_t packed_stride,
    const float* __restrict__ cen_g, float* __restrict__ out, int64_t out_stride) {
  __shared__ float cen[16];
  if (threadIdx.x < (1 << BITS)) cen[threadIdx.x] = cen_g[threadIdx.x];
  __syncthreads();
  const int64_t total = n * d;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = i / d;
    const int dim = (int)(i - row * d);
    const uint8_t* pr = packed + row * packed_stride;
    const uint32_t c = akv_stream_code<BITS>(dim, [&](int o) { return (uint32_t)pr[o]; });
    out[row * out_stride + dim] = cen[c];
  }
}

static inline int akv_grid_for(int64_t work_items, int block) {
  int64_t g = (work_items + block - 1) / block;
  int cus = akv_cached_cu_count();
  int64_t cap = (int64_t)(cus > 0 ? cus : 256) * 8;
  if (g > cap) g = cap;
  if (g < 1) g = 1;
  return (int)g;
}

extern "C" int akv_quantize_pack(const float* y, int64_t n, int d, int64_t y_stride,
                                 const float* boundaries, int bits, uint8_t* out,
                                 int64_t out_stride, void* stream) {
  AKV_REQUIRE(n >= 0 && d > 0 && d % 8 == 0, "akv_quantize_pack: bad n=%lld d=%d", (long long)n, d);
  AKV_REQUIRE(bits >= 2 && bits <= 4, "akv_quantize_pack: bits=%d not in {2,3,4}", bits);
  if (n == 0) return AKV_OK;
  AKV_REQUIRE(y && boundaries && out, "akv_quantize_pack: null pointer");
  const int grid = akv_grid_for(n * akv_packed_size(d, bits), 256);
  hipStream_t s = (hipStream_t)stream;
  if (bits == 4) akv_quantize_pack_kernel<4><<<grid, 256, 0, s>>>(y, n, d, y_stride, boundaries, out, out_stride);
  else if (bits == 3) akv_quantize_pack_kernel<3><<<grid, 256, 0, s>>>(y, n, d, y_stride, boundaries, out, out_stride);
  else akv_quantize_pack_kernel<2><<<grid, 256, 0, s>>>(y, n, d, y_stride, boundaries, out, out_stride);
  AKV_LAUNCH_CHECK("akv_quantize_pack_kernel");
  return AKV_OK;
}

extern "C" int akv_unpack_lookup(const uint8_t* packed, int64_t n, int d, int64_t packed_stride,
                                 const float* centroids, int bits, float* out, int64_t out_stride,
                                 void* stream) {
  AKV_REQUIRE(n >= 0 && d > 0 && d % 8 == 0, "akv_unpack_lookup: bad n=%lld d=%d", (long long)n, d);
  AKV_REQUIRE(bits >= 2 && bits <= 4, "akv_unpack_lookup: bits=%d not in {2,3,4}", bits);
  if (n == 0) return AKV_OK;
  AKV_REQUIRE(packed && centroids && out, "akv_unpack_lookup: null pointer");
  const int grid = akv_grid_for(n * d, 256);
  hipStream_t s = (hipStream_t)stream;
  if (bits == 4) akv_unpack_lookup_kernel<4><<<grid, 256, 0, s>>>(packed, n, d, packed_stride, centroids, out, out_stride);
  else if (bits == 3) akv_unpack_lookup_kernel<3><<<grid, 256, 0, s>>>(packed, n, d, packed_stride, centroids, out, out_stride);
  else akv_unpack_lookup_kernel<2><<<grid, 256, 0, s>>>(packed, n, d, packed_stride, centroids, out, out_stride);
  AKV_LAUNCH_CHECK("akv_unpack_lookup_kernel");
  return AKV_OK;
}

// ----------------------------------------------------------------------------------
// general encode / decode: one workgroup of 4 wavefronts, each wavefront rotates VPW vectors
// at a time with lanes owning D/64 output coordinates; the matrix (Pi^T for encode, Pi for
// decode) is staged in LDS as [k][out].
// ----------------------------------------------------------------------------------
#define AKV_GEN_WAVES 4
#define AKV_GEN_VPW 8


// acc[v][i] += sum_k in[v][k] * M[k][lane*DPL + i], k in [k0, k0 + KT)
template <int D, int KT>
__device__ __forceinline__ void akv_rotate_tile(const float* __restrict__ m_lds,  // [KT][D]
                                                const float* __restrict__ in_lds, // [VPW][D]
                                                int k0, int lane,
                                                float (&acc)[AKV_GEN_VPW][D / 64]) {
  constexpr int DPL = D / 64;
#pragma unroll 2
  for (int k = 0; k < KT; k += 4) {
    float m[4][DPL];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int i = 0; i < DPL; ++i) m[kk][i] = m_lds[(k + kk) * D + lane * DPL + i];
#pragma unroll
    for (int v = 0; v < AKV_GEN_VPW; ++v) {
      const float4 u = *(const float4*)(in_lds + v * D + k0 + k);
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        // four terms are summed on their own and then added: the running sum is rounded once per four terms
        // instead of four times (at head_dim 256 and 512 a single chain of fused multiply-adds drifted up to
        // 18 float32 units in the last place of the largest term away from the exact sum)
        const float quad = fmaf(m[0][i], u.x, fmaf(m[1][i], u.y, fmaf(m[2][i], u.z, m[3][i] * u.w)));
        acc[v][i] += quad;
      }
    }
  }
}

template <int D> struct akv_gen_cfg {
  static constexpr int KT = (D <= 128) ? D : (D == 256 ? 64 : 32);  // matrix rows staged at a time (<= 64 KiB)
  static constexpr size_t mat_floats = (size_t)KT * D;
  static constexpr size_t in_floats = (size_t)AKV_GEN_WAVES * AKV_GEN_VPW * D;
  static constexpr size_t code_bytes = (size_t)AKV_GEN_WAVES * AKV_GEN_VPW * D;
  static constexpr size_t lds_bytes = (mat_floats + in_floats) * 4 + code_bytes + 64;
};

template <int D, int BITS, int XDT, bool PAGED>
__global__ __launch_bounds__(256) void akv_encode_general_kernel(akv_gen_args a) {
  constexpr int DPL = D / 64;
  constexpr int KT = akv_gen_cfg<D>::KT;
  constexpr int P = D * BITS / 8;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  float* m_lds = (float*)lds_raw;
  float* in_lds = m_lds + akv_gen_cfg<D>::mat_floats;
  uint8_t* c_lds = (uint8_t*)(in_lds + akv_gen_cfg<D>::in_floats);
  float* bnd = (float*)(c_lds + akv_gen_cfg<D>::code_bytes);  // 16 floats

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x < (1 << BITS) - 1) bnd[threadIdx.x] = a.table[threadIdx.x];
  if (KT == D) {
    for (int i = threadIdx.x * 4; i < D * D; i += 256 * 4)
      *(float4*)(m_lds + i) = *(const float4*)(a.mat + i);
  }
  __syncthreads();

  float* my_in = in_lds + wave * AKV_GEN_VPW * D;
  uint8_t* my_c = c_lds + wave * AKV_GEN_VPW * D;
  const int64_t tile_vecs = AKV_GEN_WAVES * AKV_GEN_VPW;
  const int64_t num_tiles = (a.n + tile_vecs - 1) / tile_vecs;

  for (int64_t tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
    const int64_t base = tile * tile_vecs + wave * AKV_GEN_VPW;
    float nrm[AKV_GEN_VPW];
    // 1) load, norm, normalise
#pragma unroll
    for (int v = 0; v < AKV_GEN_VPW; ++v) {
      const int64_t n = base + v;
      float xv[DPL];
      float ss = 0.f;
      if (n < a.n) {
        const int64_t off = PAGED ? (n / a.heads) * a.xs0 + (n % a.heads) * a.xs1 : n * a.xs0;
#pragma unroll
        for (int i = 0; i < DPL; ++i) {
          xv[i] = akv_elem<XDT>::load(a.x, off + lane * DPL + i);
          ss = fmaf(xv[i], xv[i], ss);
        }
      } else {
#pragma unroll
        for (int i = 0; i < DPL; ++i) xv[i] = 0.f;
      }
      ss = akv_wave_sum(ss);
      nrm[v] = sqrtf(ss);
      const float den = nrm[v] + 1e-10f;
#pragma unroll
      for (int i = 0; i < DPL; ++i) my_in[v * D + lane * DPL + i] = xv[i] / den;
    }
    // 2) rotate
    float acc[AKV_GEN_VPW][DPL];
#pragma unroll
    for (int v = 0; v < AKV_GEN_VPW; ++v)
#pragma unroll
      for (int i = 0; i < DPL; ++i) acc[v][i] = 0.f;
    if (KT == D) {
      __syncthreads();
      akv_rotate_tile<D, KT>(m_lds, my_in, 0, lane, acc);
    } else {
      for (int k0 = 0; k0 < D; k0 += KT) {
        __syncthreads();
        for (int i = threadIdx.x * 4; i < KT * D; i += 256 * 4)
          *(float4*)(m_lds + i) = *(const float4*)(a.mat + (size_t)k0 * D + i);
        __syncthreads();
        akv_rotate_tile<D, KT>(m_lds, my_in, k0, lane, acc);
      }
    }
    // 3) codebook search -> code bytes in LDS
#pragma unroll
    for (int v = 0; v < AKV_GEN_VPW; ++v)
#pragma unroll
      for (int i = 0; i < DPL; ++i)
        my_c[v * D + lane * DPL + i] = (uint8_t)akv_search<BITS>(acc[v][i], bnd);
    __syncthreads();
    // 4) pack + store
#pragma unroll
    for (int v = 0; v < AKV_GEN_VPW; ++v) {
      const int64_t n = base + v;
      if (n >= a.n) continue;
      uint8_t* prow;
      float* nptr;
      if (PAGED) {
        const int64_t tok = n / a.heads, head = n % a.heads;
        const int64_t slot = akv_load_index(a.slots, a.slot_itype, tok);
        if (slot < 0) continue;
        const int64_t blk = slot / a.block_size, pos = slot % a.block_size;
        if (blk >= a.max_blocks) continue;
        prow = a.packed + blk * a.ps0 + pos * a.ps1 + head * a.ps2;
        nptr = a.norms + blk * a.ns0 + pos * a.ns1 + head * a.ns2;
      } else {
        prow = a.packed + n * a.ps0;
        nptr = a.norms + n;
      }
      const uint8_t* cv = my_c + v * D;
      for (int k = lane; k < P; k += 64)
        prow[k] = (uint8_t)akv_stream_byte<BITS>(k, [&](int dim) { return (uint32_t)cv[dim]; });
      if (lane == 0) *nptr = nrm[v];
    }
    __syncthreads();
  }
}

// Row n of a block-wise decode is (listed block n / (block_size*heads), position, head); false
// when the listed block id is outside the cache.  Offsets: packed in bytes, norms / output in elements.
__device__ __forceinline__ bool akv_block_row(const akv_gen_args& a, int64_t n, int64_t& po, int64_t& no, int64_t& oo) {
  const int64_t per_blk = (int64_t)a.block_size * a.heads;
  const int64_t li = n / per_blk, rem = n - li * per_blk;
  const int64_t pos = rem / a.heads, head = rem - pos * a.heads;
  const int64_t blk = akv_load_index(a.slots, a.slot_itype, li);
  if (blk < 0 || blk >= a.max_blocks) return false;
  po = blk * a.ps0 + pos * a.ps1 + head * a.ps2;
  no = blk * a.ns0 + pos * a.ns1 + head * a.ns2;
  oo = blk * a.os0 + pos * a.os1 + head * a.os2;
  return true;
}

template <int D, int BITS, int ODT, bool BLOCKS>
__global__ __launch_bounds__(256) void akv_decode_general_kernel(akv_gen_args a) {
  constexpr int DPL = D / 64;
  constexpr int KT = akv_gen_cfg<D>::KT;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  float* m_lds = (float*)lds_raw;
  float* in_lds = m_lds + akv_gen_cfg<D>::mat_floats;
  uint8_t* c_lds = (uint8_t*)(in_lds + akv_gen_cfg<D>::in_floats);
  float* cen = (float*)(c_lds + akv_gen_cfg<D>::code_bytes);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x < (1 << BITS)) cen[threadIdx.x] = a.table[threadIdx.x];
  if (KT == D) {
    for (int i = threadIdx.x * 4; i < D * D; i += 256 * 4)
      *(float4*)(m_lds + i) = *(const float4*)(a.mat + i);
  }
  __syncthreads();

  float* my_in = in_lds + wave * AKV_GEN_VPW * D;
  const int64_t tile_vecs = AKV_GEN_WAVES * AKV_GEN_VPW;
  const int64_t num_tiles = (a.n + tile_vecs - 1) / tile_vecs;

  for (int64_t tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
    const int64_t base = tile * tile_vecs + wave * AKV_GEN_VPW;
    bool live[AKV_GEN_VPW];
    int64_t noff[AKV_GEN_VPW], ooff[AKV_GEN_VPW];
#pragma unroll
    for (int v = 0; v < AKV_GEN_VPW; ++v) {
      const int64_t n = base + v;
      int64_t poff = 0;
      live[v] = n < a.n;
      if constexpr (BLOCKS) {
        noff[v] = ooff[v] = 0;
        if (live[v]) live[v] = akv_block_row(a, n, poff, noff[v], ooff[v]);
      } else {
        poff = (live[v] ? n : 0) * a.ps0; noff[v] = n; ooff[v] = n * a.os0;
      }
      const uint8_t* prow = a.packed + poff;
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        float val = 0.f;
        if (live[v]) {
          const uint32_t c = akv_stream_code<BITS>(lane * DPL + i, [&](int o) { return (uint32_t)prow[o]; });
          val = cen[c];
        }
        my_in[v * D + lane * DPL + i] = val;
      }
    }
    float acc[AKV_GEN_VPW][DPL];
#pragma unroll
    for (int v = 0; v < AKV_GEN_VPW; ++v)
#pragma unroll
      for (int i = 0; i < DPL; ++i) acc[v][i] = 0.f;
    if (KT == D) {
      __syncthreads();
      akv_rotate_tile<D, KT>(m_lds, my_in, 0, lane, acc);
    } else {
      for (int k0 = 0; k0 < D; k0 += KT) {
        __syncthreads();
        for (int i = threadIdx.x * 4; i < KT * D; i += 256 * 4)
          *(float4*)(m_lds + i) = *(const float4*)(a.mat + (size_t)k0 * D + i);
        __syncthreads();
        akv_rotate_tile<D, KT>(m_lds, my_in, k0, lane, acc);
      }
    }
#pragma unroll
    for (int v = 0; v < AKV_GEN_VPW; ++v) {
      if (!live[v]) continue;
      const float nv = a.norms[noff[v]];
#pragma unroll
      for (int i = 0; i < DPL; ++i)
        akv_elem<ODT>::store(a.out, ooff[v] + lane * DPL + i, acc[v][i] * nv);
    }
    __syncthreads();
  }
}

template <typename K>
static int akv_launch_gen(K kernel, const char* name, size_t lds, const akv_gen_args& a, void* stream) {
  static thread_local const void* configured[64];
  static thread_local int nconf = 0;
  bool seen = false;
  for (int i = 0; i < nconf; ++i) seen |= (configured[i] == (const void*)kernel);
  if (!seen) {
    AKV_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    if (nconf < 64) configured[nconf++] = (const void*)kernel;
  }
  const int64_t tile_vecs = AKV_GEN_WAVES * AKV_GEN_VPW;
  int64_t tiles = (a.n + tile_vecs - 1) / tile_vecs;
  int cus = akv_cached_cu_count();
  int64_t cap = (int64_t)(cus > 0 ? cus : 256) * 2;
  int grid = (int)(tiles < cap ? tiles : cap);
  akv_profile_mark_begin((hipStream_t)stream);
  kernel<<<grid, 256, lds, (hipStream_t)stream>>>(a);
  akv_profile_mark_end((hipStream_t)stream);
  AKV_LAUNCH_CHECK(name);
  return AKV_OK;
}

template <int D, int BITS, bool PAGED>
static int akv_encode_dispatch_dtype(int dt, const akv_gen_args& a, void* stream) {
  const size_t lds = akv_gen_cfg<D>::lds_bytes;
  switch (dt) {
    case AKV_F16: return akv_launch_gen(akv_encode_general_kernel<D, BITS, AKV_F16, PAGED>, "akv_encode_general_kernel", lds, a, stream);
    case AKV_BF16: return akv_launch_gen(akv_encode_general_kernel<D, BITS, AKV_BF16, PAGED>, "akv_encode_general_kernel", lds, a, stream);
    default: return akv_launch_gen(akv_encode_general_kernel<D, BITS, AKV_F32, PAGED>, "akv_encode_general_kernel", lds, a, stream);
  }
}

template <bool PAGED>
static int akv_encode_dispatch(int d, int bits, int dt, const akv_gen_args& a, void* stream) {
#define AKV_CASE(DD, BB) \
  if (d == DD && bits == BB) return akv_encode_dispatch_dtype<DD, BB, PAGED>(dt, a, stream);
  AKV_CASE(64, 2) AKV_CASE(64, 3) AKV_CASE(64, 4)
  AKV_CASE(128, 2) AKV_CASE(128, 3) AKV_CASE(128, 4)
  AKV_CASE(256, 2) AKV_CASE(256, 3) AKV_CASE(256, 4)
  AKV_CASE(512, 2) AKV_CASE(512, 3) AKV_CASE(512, 4)
#undef AKV_CASE
  return akv_fail(AKV_ERR_UNSUPPORTED, "encode: no kernel for head_dim=%d bits=%d", d, bits);
}

// MFMA fast path (akv_encode_mfma.hip); returns AKV_ERR_UNSUPPORTED when it does not apply.
int akv_encode_mfma_try(const akv_gen_args& a, bool paged, int x_dtype, int d, int bits,
                        const void* rot_prep, hipStream_t stream);

static int akv_check_codec_args(const char* fn, int d, int bits) {
  if (!(d == 64 || d == 128 || d == 256 || d == 512))
    return akv_fail(AKV_ERR_UNSUPPORTED, "%s: head_dim=%d not in {64,128,256,512}", fn, d);
  if (bits < 2 || bits > 4) return akv_fail(AKV_ERR_INVALID, "%s: bits=%d not in {2,3,4}", fn, bits);
  return AKV_OK;
}

extern "C" int akv_encode(const void* x, int x_dtype, int64_t n, int d, int64_t x_stride,
                          const void* rot_prep, const float* boundaries, int bits,
                          uint8_t* out_packed, int64_t packed_stride, float* out_norms,
                          void* stream) {
  AKV_REQUIRE(n >= 0, "akv_encode: n=%lld", (long long)n);
  AKV_REQUIRE(akv_valid_dtype(x_dtype), "akv_encode: bad dtype %d", x_dtype);
  int rc = akv_check_codec_args("akv_encode", d, bits);
  if (rc) return rc;
  if (n == 0) return AKV_OK;
  AKV_REQUIRE(x && rot_prep && boundaries && out_packed && out_norms, "akv_encode: null pointer");
  AKV_REQUIRE(x_stride >= d && packed_stride >= akv_packed_size(d, bits), "akv_encode: stride smaller than row");
  akv_gen_args a = {};
  a.x = x; a.n = n; a.xs0 = x_stride; a.heads = 1;
  a.mat = (const float*)rot_prep + (size_t)d * d;  // Pi^T: [k = input coord][out coord]
  a.table = boundaries;
  a.packed = out_packed; a.ps0 = packed_stride;
  a.norms = out_norms;
  rc = akv_encode_mfma_try(a, false, x_dtype, d, bits, rot_prep, (hipStream_t)stream);
  if (rc != AKV_ERR_UNSUPPORTED) return rc;
  return akv_encode_dispatch<false>(d, bits, x_dtype, a, stream);
}

extern "C" int akv_encode_paged_kv(const void* k, const void* v, int x_dtype, int64_t num_tokens,
                                   int num_kv_heads, int d, int64_t xs_token, int64_t xs_head,
                                   const void* slot_mapping, int slot_itype, const void* rot_prep,
                                   const float* boundaries, int bits, uint8_t* k_packed, uint8_t* v_packed,
                                   int64_t ps_blk, int64_t ps_pos, int64_t ps_head, float* k_norms,
                                   float* v_norms, int64_t ns_blk, int64_t ns_pos, int64_t ns_head,
                                   int block_size, int64_t max_blocks, void* stream) {
  AKV_REQUIRE(num_tokens >= 0 && num_kv_heads > 0, "akv_encode_paged_kv: bad sizes");
  AKV_REQUIRE(akv_valid_dtype(x_dtype) && akv_valid_itype(slot_itype), "akv_encode_paged_kv: bad dtype");
  AKV_REQUIRE(block_size > 0 && max_blocks >= 0, "akv_encode_paged_kv: bad block_size/max_blocks");
  int rc = akv_check_codec_args("akv_encode_paged_kv", d, bits);
  if (rc) return rc;
  if (num_tokens == 0 || max_blocks == 0) return AKV_OK;
  AKV_REQUIRE(k && v && slot_mapping && rot_prep && boundaries && k_packed && v_packed && k_norms && v_norms,
              "akv_encode_paged_kv: null pointer");
  akv_gen_args a = {};
  a.x = k; a.n = num_tokens * num_kv_heads; a.xs0 = xs_token; a.xs1 = xs_head; a.heads = num_kv_heads;
  a.slots = slot_mapping; a.slot_itype = slot_itype; a.block_size = block_size; a.max_blocks = max_blocks;
  a.mat = (const float*)rot_prep + (size_t)d * d;
  a.table = boundaries;
  a.packed = k_packed; a.ps0 = ps_blk; a.ps1 = ps_pos; a.ps2 = ps_head;
  a.norms = k_norms; a.ns0 = ns_blk; a.ns1 = ns_pos; a.ns2 = ns_head;
  a.x2 = v; a.packed2 = v_packed; a.norms2 = v_norms;
  rc = akv_encode_mfma_try(a, true, x_dtype, d, bits, rot_prep, (hipStream_t)stream);
  if (rc != AKV_ERR_UNSUPPORTED) return rc;
  // layouts the matrix-core kernel does not take: one launch per tensor
  akv_gen_args b = a;
  a.x2 = nullptr; a.packed2 = nullptr; a.norms2 = nullptr;
  b.x = v; b.packed = v_packed; b.norms = v_norms; b.x2 = nullptr; b.packed2 = nullptr; b.norms2 = nullptr;
  rc = akv_encode_dispatch<true>(d, bits, x_dtype, a, stream);
  if (rc) return rc;
  return akv_encode_dispatch<true>(d, bits, x_dtype, b, stream);
}

extern "C" int akv_encode_paged(const void* x, int x_dtype, int64_t num_tokens, int num_kv_heads,
                                int d, int64_t xs_token, int64_t xs_head, const void* slot_mapping,
                                int slot_itype, const void* rot_prep, const float* boundaries,
                                int bits, uint8_t* out_packed, int64_t ps_blk, int64_t ps_pos,
                                int64_t ps_head, float* out_norms, int64_t ns_blk, int64_t ns_pos,
                                int64_t ns_head, int block_size, int64_t max_blocks, void* stream) {
  AKV_REQUIRE(num_tokens >= 0 && num_kv_heads > 0, "akv_encode_paged: bad sizes");
  AKV_REQUIRE(akv_valid_dtype(x_dtype) && akv_valid_itype(slot_itype), "akv_encode_paged: bad dtype");
  AKV_REQUIRE(block_size > 0 && max_blocks >= 0, "akv_encode_paged: bad block_size/max_blocks");
  int rc = akv_check_codec_args("akv_encode_paged", d, bits);
  if (rc) return rc;
  if (num_tokens == 0 || max_blocks == 0) return AKV_OK;
  AKV_REQUIRE(x && slot_mapping && rot_prep && boundaries && out_packed && out_norms,
              "akv_encode_paged: null pointer");
  akv_gen_args a = {};
  a.x = x; a.n = num_tokens * num_kv_heads; a.xs0 = xs_token; a.xs1 = xs_head; a.heads = num_kv_heads;
  a.slots = slot_mapping; a.slot_itype = slot_itype; a.block_size = block_size; a.max_blocks = max_blocks;
  a.mat = (const float*)rot_prep + (size_t)d * d;
  a.table = boundaries;
  a.packed = out_packed; a.ps0 = ps_blk; a.ps1 = ps_pos; a.ps2 = ps_head;
  a.norms = out_norms; a.ns0 = ns_blk; a.ns1 = ns_pos; a.ns2 = ns_head;
  rc = akv_encode_mfma_try(a, true, x_dtype, d, bits, rot_prep, (hipStream_t)stream);
  if (rc != AKV_ERR_UNSUPPORTED) return rc;
  return akv_encode_dispatch<true>(d, bits, x_dtype, a, stream);
}

template <int D, int BITS, bool BLOCKS>
static int akv_decode_dispatch_dtype(int dt, const akv_gen_args& a, void* stream) {
  const size_t lds = akv_gen_cfg<D>::lds_bytes;
  switch (dt) {
    case AKV_F16: return akv_launch_gen(akv_decode_general_kernel<D, BITS, AKV_F16, BLOCKS>, "akv_decode_general_kernel", lds, a, stream);
    case AKV_BF16: return akv_launch_gen(akv_decode_general_kernel<D, BITS, AKV_BF16, BLOCKS>, "akv_decode_general_kernel", lds, a, stream);
    default: return akv_launch_gen(akv_decode_general_kernel<D, BITS, AKV_F32, BLOCKS>, "akv_decode_general_kernel", lds, a, stream);
  }
}

template <bool BLOCKS>
static int akv_decode_dispatch(int d, int bits, int out_dtype, const akv_gen_args& a, void* stream) {
#define AKV_CASE(DD, BB) \
  if (d == DD && bits == BB) return akv_decode_dispatch_dtype<DD, BB, BLOCKS>(out_dtype, a, stream);
  AKV_CASE(64, 2) AKV_CASE(64, 3) AKV_CASE(64, 4)
  AKV_CASE(128, 2) AKV_CASE(128, 3) AKV_CASE(128, 4)
  AKV_CASE(256, 2) AKV_CASE(256, 3) AKV_CASE(256, 4)
  AKV_CASE(512, 2) AKV_CASE(512, 3) AKV_CASE(512, 4)
#undef AKV_CASE
  return akv_fail(AKV_ERR_UNSUPPORTED, "decode: no kernel for head_dim=%d bits=%d", d, bits);
}

extern "C" int akv_decode(const uint8_t* packed, int64_t packed_stride, const float* norms,
                          int64_t n, int d, const void* rot_prep, const float* centroids, int bits,
                          void* out, int out_dtype, int64_t out_stride, void* stream) {
  AKV_REQUIRE(n >= 0, "akv_decode: n=%lld", (long long)n);
  AKV_REQUIRE(akv_valid_dtype(out_dtype), "akv_decode: bad dtype %d", out_dtype);
  int rc = akv_check_codec_args("akv_decode", d, bits);
  if (rc) return rc;
  if (n == 0) return AKV_OK;
  AKV_REQUIRE(packed && norms && rot_prep && centroids && out, "akv_decode: null pointer");
  AKV_REQUIRE(out_stride >= d && packed_stride >= akv_packed_size(d, bits), "akv_decode: stride smaller than row");
  akv_gen_args a = {};
  a.n = n;
  a.mat = (const float*)rot_prep;  // Pi: [k = rotated coord][out coord]
  a.table = centroids;
  a.packed = const_cast<uint8_t*>(packed); a.ps0 = packed_stride;
  a.norms = const_cast<float*>(norms);
  a.out = out; a.os0 = out_stride;
  rc = akv_decode_mfma_try(a, false, d, bits, out_dtype, rot_prep, (hipStream_t)stream);
  if (rc != AKV_ERR_UNSUPPORTED) return rc;
  return akv_decode_dispatch<false>(d, bits, out_dtype, a, stream);
}

// Decode of whole cache blocks in place of the reference's gather + decode + scatter
// (aither_kvcache/vllm/backend.py:1040-1091): every block id in `block_ids` that lies in
// [0, num_blocks) is decoded from the packed cache into the block of the same index of `out`.
extern "C" int akv_decode_blocks(const uint8_t* packed, int64_t ps_blk, int64_t ps_pos, int64_t ps_head,
                                 const float* norms, int64_t ns_blk, int64_t ns_pos, int64_t ns_head,
                                 const void* block_ids, int ids_itype, int64_t num_ids, int64_t num_blocks,
                                 int block_size, int num_kv_heads, int d, const void* rot_prep,
                                 const float* centroids, int bits, void* out, int out_dtype, int64_t os_blk,
                                 int64_t os_pos, int64_t os_head, void* stream) {
  AKV_REQUIRE(num_ids >= 0 && num_blocks >= 0 && block_size > 0 && num_kv_heads > 0, "akv_decode_blocks: bad sizes");
  AKV_REQUIRE(akv_valid_dtype(out_dtype) && akv_valid_itype(ids_itype), "akv_decode_blocks: bad dtype");
  int rc = akv_check_codec_args("akv_decode_blocks", d, bits);
  if (rc) return rc;
  if (num_ids == 0 || num_blocks == 0) return AKV_OK;
  AKV_REQUIRE(packed && norms && block_ids && rot_prep && centroids && out, "akv_decode_blocks: null pointer");
  akv_gen_args a = {};
  a.n = num_ids * block_size * num_kv_heads;
  a.heads = num_kv_heads; a.block_size = block_size; a.max_blocks = num_blocks;
  a.slots = block_ids; a.slot_itype = ids_itype;
  a.mat = (const float*)rot_prep;
  a.table = centroids;
  a.packed = const_cast<uint8_t*>(packed); a.ps0 = ps_blk; a.ps1 = ps_pos; a.ps2 = ps_head;
  a.norms = const_cast<float*>(norms); a.ns0 = ns_blk; a.ns1 = ns_pos; a.ns2 = ns_head;
  a.out = out; a.os0 = os_blk; a.os1 = os_pos; a.os2 = os_head;
  rc = akv_decode_mfma_try(a, true, d, bits, out_dtype, rot_prep, (hipStream_t)stream);
  if (rc != AKV_ERR_UNSUPPORTED) return rc;
  return akv_decode_dispatch<true>(d, bits, out_dtype, a, stream);
}
