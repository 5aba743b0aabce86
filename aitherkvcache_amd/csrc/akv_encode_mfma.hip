// MFMA encode (norm -> rotate -> codebook search -> pack -> store) for float16 input at head_dim 128.
//
// The rotation is the only heavy arithmetic of the encode path (128 x 128 multiply-adds per
// vector), so it runs on the matrix cores; everything else is arranged so that the matrix-core
// register layouts are also the memory layouts:
//
//   Y[v, j] = sum_i X[v, i] * Pi[j, i]                     v_mfma_f32_16x16x32_f16
//     A = X: lane (row = l%16, g = l/16) holds, for k-step ks, elements i = 32g + 8ks + e (e<8)
//         of vector `row` -- 64 contiguous bytes of the input row, loaded by four 16-byte loads
//         that ARE the four A operands.  float16 input is exact in the operand, so the vector is
//         not normalised before the product: y = (sum_i Pi[j,i] x_i) * 1/(|x| + 1e-10), with one
//         correctly rounded reciprocal per vector.
//     B = Pi: float32 entries split into two float16 terms (hi + lo, scaled by 64 to stay clear
//         of float16 subnormals), i.e. two MFMAs per tile and ~22 bits of the matrix.  N-tile nt,
//         column col is output coordinate j = 8 col + nt.
//     D: lane (col, g) holds rows 4g..4g+3; over the eight N-tiles it collects outputs
//         8col..8col+7 of a vector: one dword of a 4-bit row, three bytes of a 3-bit row, one
//         halfword of a 2-bit row -- sixteen lanes write one packed row contiguously.
//
// Codebook search: code = #{b < y}.  A table of EM_CELLS uniform cells over the boundary range
// maps cell -> (number of boundaries in lower cells, the one boundary inside the cell or +inf);
// the cell index is a monotone function of y evaluated by the same instructions for y and, when
// the table is built, for the boundaries, so base + (boundary < y) is exact for every float.
// If two boundaries share a cell (no such codebook is produced by the library) the kernel falls
// back to counting all boundaries.
//
// A wavefront encodes 64 vectors per step (four M-tiles share every B operand read from LDS);
// a workgroup is eight independent wavefronts plus the B operand (64 KB) and the cell table.
#include "akv_common.h"

typedef _Float16 em_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 em_half2 __attribute__((ext_vector_type(2)));
typedef float em_float4 __attribute__((ext_vector_type(4)));

#define EM_WAVES 8
#define EM_THREADS (EM_WAVES * 64)
#define EM_ROWS 64                 // vectors per wavefront step
#define EM_CELLS 128
#define EM_PSCALE 64.f             // scale of the matrix operand
#define EM_B_BYTES 65536           // [hi/lo][8 nt][4 ks][64 lanes] x 16 B
#define EM_LUT_OFF EM_B_BYTES      // EM_CELLS x {uint32 base, float boundary}
#define EM_PAR_OFF (EM_LUT_OFF + EM_CELLS * 8)   // float inv_w, float off, uint32 bad, pad
#define EM_BND_OFF (EM_PAR_OFF + 16)              // 16 floats: boundaries (fallback search)
#define EM_WAVE_OFF (EM_BND_OFF + 64)
#define EM_WAVE_BYTES (EM_ROWS * (8 + 8 + 8 + 4))  // src offset, packed offset, norm offset, 1/(|x|+eps)
#define EM_LDS_BYTES (EM_WAVE_OFF + EM_WAVES * EM_WAVE_BYTES)

// ----------------------------------------------------------------------------------
// B operand: prep + 2*d*d floats (the reserved half of the prepared-rotation buffer)
// ----------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void akv_em_prepare_kernel(const float* __restrict__ Pi, uint4* __restrict__ bop) {
  // one thread per (nt, ks, lane): 8 entries, hi and lo
  const int t = blockIdx.x * 256 + threadIdx.x;      // 8*4*64 = 2048 threads
  const int lane = t & 63, ks = (t >> 6) & 3, nt = t >> 8;
  const int col = lane & 15, g = lane >> 4;
  const int j = 8 * col + nt;
  uint32_t hi[4], lo[4];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float v = Pi[(size_t)j * 128 + 32 * g + 8 * ks + e] * EM_PSCALE;
    const __half h = __float2half_rn(v);
    const __half l = __float2half_rn(v - __half2float(h));
    if (e & 1) {
      hi[e >> 1] |= (uint32_t)__half_as_ushort(h) << 16;
      lo[e >> 1] |= (uint32_t)__half_as_ushort(l) << 16;
    } else {
      hi[e >> 1] = __half_as_ushort(h);
      lo[e >> 1] = __half_as_ushort(l);
    }
  }
  bop[t] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
  bop[2048 + t] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
}

int akv_prepare_rotation_mfma(const float* rotation, int d, void* prep, hipStream_t stream) {
  if (d != 128) return AKV_OK;
  uint4* bop = (uint4*)((float*)prep + (size_t)2 * d * d);
  akv_em_prepare_kernel<<<8, 256, 0, stream>>>(rotation, bop);
  AKV_LAUNCH_CHECK("akv_em_prepare_kernel");
  return AKV_OK;
}

// ----------------------------------------------------------------------------------
// encode kernel
// ----------------------------------------------------------------------------------
typedef uint32_t em_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t em_u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) em_u32x4 em_lds_u128;
typedef __attribute__((address_space(3))) em_u32x2 em_lds_u64;

// cell of a value: monotone non-decreasing in y for inv_w > 0
__device__ __forceinline__ uint32_t em_cell(float y, float inv_w, float off) {
  const float t = __builtin_amdgcn_fmed3f(fmaf(y, inv_w, off), 0.f, (float)(EM_CELLS - 1));
  return (uint32_t)t;
}

template <int BITS, bool PAGED>
__global__ __launch_bounds__(EM_THREADS) void akv_encode_mfma_kernel(akv_gen_args a, const uint4* __restrict__ bop) {
  extern __shared__ __align__(16) unsigned char lds[];
  constexpr int NB = (1 << BITS) - 1;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 15, g = lane >> 4;

  // ---- workgroup set-up: B operand, boundaries, cell table
  {
    uint4* b_lds = (uint4*)lds;
    for (int i = threadIdx.x; i < EM_B_BYTES / 16; i += EM_THREADS) b_lds[i] = bop[i];
    float* bnd = (float*)(lds + EM_BND_OFF);
    if (threadIdx.x < 16) bnd[threadIdx.x] = threadIdx.x < NB ? a.table[threadIdx.x] : INFINITY;
    __syncthreads();
    float* par = (float*)(lds + EM_PAR_OFF);
    if (threadIdx.x == 0) {
      const float lo = bnd[0], hi = bnd[NB - 1];
      const float w = (hi - lo) / (float)(EM_CELLS - 2);
      const float inv_w = 1.f / w;
      par[0] = inv_w;
      par[1] = 1.f - lo * inv_w;       // boundary 0 falls in cell 1
      // usable only for finite, strictly increasing boundaries
      bool ok = (w > 0.f) && (inv_w < INFINITY);
      for (int k = 1; k < NB; ++k) ok = ok && (bnd[k] > bnd[k - 1]);
      ((uint32_t*)par)[2] = ok ? 0u : 1u;
    }
    __syncthreads();
    const float inv_w = par[0], off = par[1];
    if (threadIdx.x < EM_CELLS) {
      uint32_t base = 0, cnt = 0;
      float inside = INFINITY;
      for (int k = 0; k < NB; ++k) {
        const uint32_t c = em_cell(bnd[k], inv_w, off);
        if (c < threadIdx.x) ++base;
        if (c == threadIdx.x) { ++cnt; inside = bnd[k]; }
      }
      uint32_t* lut = (uint32_t*)(lds + EM_LUT_OFF);
      lut[2 * threadIdx.x] = base;
      lut[2 * threadIdx.x + 1] = __float_as_uint(inside);
      if (cnt > 1) atomicOr((uint32_t*)par + 2, 1u);
    }
    __syncthreads();
  }
  const float inv_w = ((const float*)(lds + EM_PAR_OFF))[0];
  const float off = ((const float*)(lds + EM_PAR_OFF))[1];
  const bool linear_search = ((const uint32_t*)(lds + EM_PAR_OFF))[2] != 0;   // uniform
  const float* bnd = (const float*)(lds + EM_BND_OFF);
  const uint32_t lut_addr = EM_LUT_OFF;

  unsigned char* wl = lds + EM_WAVE_OFF + wave * EM_WAVE_BYTES;
  int64_t* src_off = (int64_t*)wl;                    // element offset of the vector in x, or -1
  int64_t* dst_p = (int64_t*)(wl + EM_ROWS * 8);      // byte offset of the packed row, or -1
  int64_t* dst_n = (int64_t*)(wl + EM_ROWS * 16);     // element offset of the norm
  float* rinv = (float*)(wl + EM_ROWS * 24);          // 1/(|x| + 1e-10), scaled back by 1/EM_PSCALE; NaN rows flagged

  const int64_t steps = (a.n + EM_ROWS - 1) / EM_ROWS;
  for (int64_t step = (int64_t)blockIdx.x * EM_WAVES + wave; step < steps; step += (int64_t)gridDim.x * EM_WAVES) {
    const int64_t base = step * EM_ROWS;
    // ---- lane l resolves the addresses of vector base + l
    {
      const int64_t n = base + lane;
      int64_t so = -1, dp = -1, dn = 0;
      if (n < a.n) {
        if (PAGED) {
          const int64_t tok = n / a.heads, head = n - tok * a.heads;
          so = tok * a.xs0 + head * a.xs1;
          const int64_t slot = akv_load_index(a.slots, a.slot_itype, tok);
          if (slot >= 0) {
            const int64_t blk = slot / a.block_size, pos = slot - blk * a.block_size;
            if (blk < a.max_blocks) {
              dp = blk * a.ps0 + pos * a.ps1 + head * a.ps2;
              dn = blk * a.ns0 + pos * a.ns1 + head * a.ns2;
            }
          }
        } else {
          so = n * a.xs0;
          dp = n * a.ps0;
          dn = n;
        }
      }
      src_off[lane] = so;
      dst_p[lane] = dp;
      dst_n[lane] = dn;
    }
    // ---- A operands straight from memory; squared norms
    em_half8 A[4][4];
    float ss[4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      const int64_t so = src_off[16 * mt + (lane & 15)];
      ss[mt] = 0.f;
      if (so >= 0) {
        const uint4* p = (const uint4*)((const __half*)a.x + so + 32 * g);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          union { uint4 u; em_half8 h; em_half2 h2[4]; } cv;
          cv.u = p[ks];
          A[mt][ks] = cv.h;
        }
      } else {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) A[mt][ks] = (em_half8){0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        union { em_half8 h; em_half2 h2[4]; } cv;
        cv.h = A[mt][ks];
#pragma unroll
        for (int q = 0; q < 4; ++q) ss[mt] = __builtin_amdgcn_fdot2(cv.h2[q], cv.h2[q], ss[mt], false);
      }
      ss[mt] += __shfl_xor(ss[mt], 16, 64);
      ss[mt] += __shfl_xor(ss[mt], 32, 64);
    }
    // lane (row, g = mt) finishes vector 16 mt + row: norm out, reciprocal to LDS
    {
      float mine = ss[0];
      if (g == 1) mine = ss[1];
      if (g == 2) mine = ss[2];
      if (g == 3) mine = ss[3];
      const float nrm = sqrtf(mine);
      const float r = (1.f / (nrm + 1e-10f)) * (1.f / EM_PSCALE);
      // a vector with a NaN or an infinity rotates to NaN everywhere: every code is the last level
      rinv[lane] = (nrm < INFINITY) ? r : __uint_as_float(0x7fc00000u);
      if (dst_p[lane] >= 0) a.norms[dst_n[lane]] = nrm;
    }
    // ---- rotate, search, pack
    uint32_t packed[4][4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) packed[mt][i] = 0u;
    em_float4 rv[4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
      union { em_u32x4 u; em_float4 f; } cv;
      cv.u = *(em_lds_u128*)(uintptr_t)(uint32_t)(EM_WAVE_OFF + wave * EM_WAVE_BYTES + EM_ROWS * 24 + (16 * mt + 4 * g) * 4);
      rv[mt] = cv.f;
    }
#pragma unroll
    for (int nt = 0; nt < 8; ++nt) {
      em_float4 acc[4];
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) acc[mt] = (em_float4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        union { em_u32x4 u; em_half8 h; } bh, bl;
        bh.u = *(em_lds_u128*)(uintptr_t)(uint32_t)(((nt * 4 + ks) * 64 + lane) * 16);
        bl.u = *(em_lds_u128*)(uintptr_t)(uint32_t)(32768 + ((nt * 4 + ks) * 64 + lane) * 16);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[mt][ks], bh.h, acc[mt], 0, 0, 0);
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[mt][ks], bl.h, acc[mt], 0, 0, 0);
        }
      }
      // output coordinate 8 col + nt of rows 4g + i
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float y = acc[mt][i] * rv[mt][i];
          uint32_t code;
          if (!linear_search) {
            const uint32_t c = em_cell(y, inv_w, off);
            const em_u32x2 e = *(em_lds_u64*)(uintptr_t)(lut_addr + c * 8u);
            code = e.x + ((__uint_as_float(e.y) < y) ? 1u : 0u);
          } else {
            code = akv_search<BITS>(y, bnd);
          }
          // position of code nt inside the lane's packed group of eight codes
          const int sh = BITS == 4 ? 8 * (nt >> 1) + ((nt & 1) ? 0 : 4)
                       : BITS == 3 ? 21 - 3 * nt
                                   : 8 * (nt >> 2) + 6 - 2 * (nt & 3);
          packed[mt][i] |= code << sh;
        }
    }
    // ---- store: lane (col, g) writes group col of rows 4g + i
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = 16 * mt + 4 * g + i;
        const int64_t dp = dst_p[row];
        if (dp < 0) continue;
        uint32_t v = packed[mt][i];
        if (!(rv[mt][i] == rv[mt][i])) v = 0xffffffffu;     // NaN vector: last level everywhere
        uint8_t* prow = a.packed + dp;
        if (BITS == 4) {
          *(uint32_t*)(prow + 4 * col) = v;
        } else if (BITS == 3) {
          prow[3 * col] = (uint8_t)(v >> 16);
          prow[3 * col + 1] = (uint8_t)(v >> 8);
          prow[3 * col + 2] = (uint8_t)v;
        } else {
          *(uint16_t*)(prow + 2 * col) = (uint16_t)v;
        }
      }
  }
}

static bool em_disabled() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("AKV_DISABLE_MFMA");
    v = (e && e[0] == '1') ? 1 : 0;
  }
  return v == 1;
}

int akv_encode_mfma_try(const akv_gen_args& a, bool paged, int x_dtype, int d, int bits,
                        const void* rot_prep, hipStream_t stream) {
  if (em_disabled() || d != 128 || x_dtype != AKV_F16) return AKV_ERR_UNSUPPORTED;
  // 16-byte loads of the input rows; aligned stores of the packed groups
  if (((uintptr_t)a.x & 15) || (a.xs0 & 7) || (paged && (a.xs1 & 7))) return AKV_ERR_UNSUPPORTED;
  const int64_t amask = bits == 4 ? 3 : bits == 2 ? 1 : 0;
  if (((uintptr_t)a.packed | (uintptr_t)a.ps0 | (uintptr_t)a.ps1 | (uintptr_t)a.ps2) & amask) return AKV_ERR_UNSUPPORTED;
  const uint4* bop = (const uint4*)((const float*)rot_prep + (size_t)2 * d * d);
  const int64_t steps = (a.n + EM_ROWS - 1) / EM_ROWS;
  const int64_t wgs = (steps + EM_WAVES - 1) / EM_WAVES;
  const int grid = (int)(wgs < akv_cached_cu_count() ? wgs : akv_cached_cu_count());
#define EM_LAUNCH(BB, PG)                                                                            \
  do {                                                                                               \
    static bool configured = false;                                                                  \
    if (!configured) {                                                                               \
      AKV_HIP(hipFuncSetAttribute((const void*)akv_encode_mfma_kernel<BB, PG>,                       \
                                  hipFuncAttributeMaxDynamicSharedMemorySize, EM_LDS_BYTES));        \
      configured = true;                                                                             \
    }                                                                                                \
    akv_profile_mark_begin(stream);                                                                  \
    akv_encode_mfma_kernel<BB, PG><<<grid, EM_THREADS, EM_LDS_BYTES, stream>>>(a, bop);              \
    akv_profile_mark_end(stream);                                                                    \
  } while (0)
  if (paged) {
    if (bits == 4) EM_LAUNCH(4, true); else if (bits == 3) EM_LAUNCH(3, true); else EM_LAUNCH(2, true);
  } else {
    if (bits == 4) EM_LAUNCH(4, false); else if (bits == 3) EM_LAUNCH(3, false); else EM_LAUNCH(2, false);
  }
#undef EM_LAUNCH
  AKV_LAUNCH_CHECK("akv_encode_mfma_kernel");
  return AKV_OK;
}
