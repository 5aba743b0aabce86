// MFMA encode (norm -> rotate -> codebook search -> pack -> store) for float16, bfloat16 and float32
// input at head_dim 128.
//
// The rotation is the only heavy arithmetic of the encode path (128 x 128 multiply-adds per
// vector), so it runs on the matrix cores; everything else is arranged so that the matrix-core
// register layouts are also the memory layouts:
//
//   Y[v, j] = sum_i X[v, i] * Pi[j, i]                     v_mfma_f32_16x16x32_f16
//     A = X: lane (row = l%16, g = l/16) holds, for k-step ks, elements i = 32g + 8ks + e (e<8)
//         of vector `row` -- 64 contiguous bytes of the input row, loaded by four 16-byte loads
//         that ARE the four A operands (measured faster than the layout in which the four lanes
//         of a row share each load).  float16 input is exact in the operand, so the vector is
//         not normalised before the product: y = (sum_i Pi[j,i] x_i) * 1/(|x| + 1e-10), with one
//         correctly rounded reciprocal per vector.  float32 input is scaled by the power of two of the
//         row's largest element and split into two float16 terms (hi + lo: every element to half a
//         float32 ulp of itself, or to 2^-25 of the largest element where lo is subnormal); the product
//         takes three MFMAs per tile (x_hi Pi_hi + x_hi Pi_lo + x_lo Pi_hi) and a wavefront step
//         holds one M-tile instead of two, so that both terms of the rows fit the registers.
//     B = Pi: float32 entries split into two float16 terms (hi + lo, scaled by 64 to stay clear
//         of float16 subnormals), i.e. two MFMAs per tile and ~22 bits of the matrix.  N-tile nt,
//         column col is output coordinate j = 8 col + nt.
//     D: lane (col, g) holds rows 4g..4g+3; over the eight N-tiles it collects outputs
//         8col..8col+7 of a vector: one dword of a 4-bit row, three bytes of a 3-bit row, one
//         halfword of a 2-bit row -- sixteen lanes write one packed row contiguously.
//
// Codebook search: code = #{b < y}.  A table of EM_CELLS uniform cells over y in (-1.004, 1.004)
// maps cell -> (number of boundaries in lower cells, the one boundary inside the cell or +inf);
// the cell index is a monotone function of y evaluated by the same instructions for y and, when
// the table is built, for the boundaries, so base + (boundary < y) is exact for every float in
// range.  |y| <= (longest row of Pi) x |unit vector|, and the prepare step records whether every
// row is short enough; if not, or if two boundaries share a cell or lie outside (-1, 1) (no such
// codebook is produced by the library), the kernel counts all boundaries instead.
//
// A wavefront encodes EM_ROWS vectors per step (its M-tiles share every B operand read from LDS);
// a workgroup is EM_WAVES independent wavefronts plus the B operand (64 KB) and the cell table.
// Vector-unit and matrix-core time add up on a SIMD here (measured), so the search is kept to six
// vector instructions per value: multiply, fma, mask, compare, add-with-carry, shift-or.
#include "akv_common.h"
#include <type_traits>

typedef _Float16 em_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 em_half2 __attribute__((ext_vector_type(2)));
typedef float em_float4 __attribute__((ext_vector_type(4)));
typedef unsigned short em_us2 __attribute__((ext_vector_type(2)));

#ifndef EM_MT
#define EM_MT 2                    // M-tiles (16 vectors each) per wavefront step
#endif
#define EM_WAVES (32 / EM_MT)      // EM_MT 2: sixteen wavefronts under 128 registers; 4: eight under 256
#define EM_THREADS (EM_WAVES * 64)
#define EM_ROWS (16 * EM_MT)       // vectors per wavefront step
#define EM_CELLS 512               // uniform cells over y in [-1.0039, 1.0039)
#define EM_CELL_S 2040.f           // 8 x cells per unit of y: the cell table is addressed in bytes
#define EM_CELL_C (8388608.f + 2048.f)   // 2^23 + centre: the sum's mantissa is 8 x the cell coordinate
#define EM_CELL_MASK 0xff8u
#define EM_MAX_ROW_NORM 1.0015f    // |y| <= |row of Pi| <= this keeps y inside the table
#define EM_PSCALE 64.f             // scale of the matrix operand
#define EM_B_BYTES 65536           // [hi/lo][8 nt][4 ks][64 lanes] x 16 B
#define EM_LUT_OFF 0               // EM_CELLS x {uint32 base, float boundary}: LDS address = cell byte offset
#define EM_B_OFF (EM_CELLS * 8)
#define EM_PAR_OFF (EM_B_OFF + EM_B_BYTES)       // uint32 bad, pad
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

// flag word after the B operand: 1 when some row of the matrix is longer than EM_MAX_ROW_NORM (then
// a rotated unit vector may leave the range of the cell table and the kernel counts boundaries)
__global__ __launch_bounds__(128) void akv_em_rownorm_kernel(const float* __restrict__ Pi, uint32_t* __restrict__ flag) {
  __shared__ uint32_t bad;
  if (threadIdx.x == 0) bad = 0u;
  __syncthreads();
  float ss = 0.f;
  for (int i = 0; i < 128; ++i) {
    const float v = Pi[(size_t)threadIdx.x * 128 + i];
    ss = fmaf(v, v, ss);
  }
  if (!(sqrtf(ss) <= EM_MAX_ROW_NORM)) atomicOr(&bad, 1u);
  __syncthreads();
  if (threadIdx.x == 0) flag[0] = bad;
}

int akv_prepare_rotation_mfma(const float* rotation, int d, void* prep, hipStream_t stream) {
  if (d != 128) return AKV_OK;
  uint4* bop = (uint4*)((float*)prep + (size_t)2 * d * d);
  akv_em_prepare_kernel<<<8, 256, 0, stream>>>(rotation, bop);
  AKV_LAUNCH_CHECK("akv_em_prepare_kernel");
  akv_em_rownorm_kernel<<<1, 128, 0, stream>>>(rotation, (uint32_t*)(bop + EM_B_BYTES / 16));
  AKV_LAUNCH_CHECK("akv_em_rownorm_kernel");
  return AKV_OK;
}

// ----------------------------------------------------------------------------------
// encode kernel
// ----------------------------------------------------------------------------------
typedef uint32_t em_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t em_u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) em_u32x4 em_lds_u128;
typedef __attribute__((address_space(3))) em_u32x2 em_lds_u64;

// Byte offset of the cell of y in the table: y * S + (2^23 + centre) has the cell coordinate (x 8)
// in its mantissa, so one fused multiply-add and one mask replace scale, clamp, convert and shift.
// Monotone non-decreasing for |y| < 1.0039; NaN lands inside the table like any other pattern.
__device__ __forceinline__ uint32_t em_cell(float y) {
  return __float_as_uint(fmaf(y, EM_CELL_S, EM_CELL_C)) & EM_CELL_MASK;
}

// MT: M-tiles (16 vectors each) per wavefront step -- MT, or 1 for float32 input
// SPLIT (calls of a few thousand vectors, e.g. one serving step): a workgroup is eight wavefronts that share ONE
// step of 16 vectors, wavefront w computes N-tile w with its eighth of the B operand straight from memory in
// registers -- no 64 KB fill, no cell table, one barrier; the codes meet in LDS and 256 threads pack and store
// them.  Same products, same reciprocal, same comparison against the boundaries: the same codes.
#define EM_SPLIT_WAVES 8
#define EM_SPLIT_CODES 0           // [16 vectors][128 coordinates] code bytes
#define EM_SPLIT_WAVE_OFF 2048
#define EM_SPLIT_LDS_BYTES (EM_SPLIT_WAVE_OFF + EM_SPLIT_WAVES * EM_WAVE_BYTES)
template <int BITS, bool PAGED, int XDT, bool DIRECT, int MT, bool SPLIT = false>
__global__ __launch_bounds__(EM_THREADS) void akv_encode_mfma_kernel(akv_gen_args a, const uint4* __restrict__ bop) {
  extern __shared__ __align__(16) unsigned char lds[];
  static_assert(MT <= MT && (XDT != AKV_F32 || MT == 1), "the LDS regions are sized for MT tiles");
  static_assert(!SPLIT || (MT == 1 && XDT != AKV_F32 && !DIRECT), "the split form: one M-tile of 16-bit rows");
  constexpr uint32_t WAVE_OFF = SPLIT ? EM_SPLIT_WAVE_OFF : EM_WAVE_OFF;
  constexpr int ROWS = 16 * MT;                       // vectors per wavefront step
  constexpr int XB = XDT == AKV_F32 ? 4 : 2;          // bytes per input element
  constexpr int NA = XDT == AKV_F32 ? 2 : 1;          // float16 terms of the input operand
  constexpr int NB = (1 << BITS) - 1;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 15, g = lane >> 4;

  // ---- workgroup set-up: B operand, boundaries, cell table (called after the wavefront has requested the rows
  // of its first step, so that their trip to memory runs beside the fill: a call of one serving step is a single
  // step per wavefront and nothing else)
  auto setup = [&]() {
    uint4* b_lds = (uint4*)(lds + EM_B_OFF);
    for (int i = threadIdx.x; i < EM_B_BYTES / 16; i += EM_THREADS) b_lds[i] = bop[i];
    float* bnd = (float*)(lds + EM_BND_OFF);
    uint32_t* par = (uint32_t*)(lds + EM_PAR_OFF);
    if (threadIdx.x < 16) bnd[threadIdx.x] = threadIdx.x < NB ? a.table[threadIdx.x] : INFINITY;
    if (threadIdx.x == 0) par[0] = ((const uint32_t*)(bop + EM_B_BYTES / 16))[0];   // rows of Pi too long for the table
    __syncthreads();
    if (threadIdx.x == 0) {
      // the table serves finite, strictly increasing boundaries inside (-1, 1)
      bool ok = fabsf(bnd[0]) < 1.f && fabsf(bnd[NB - 1]) < 1.f;
      for (int k = 1; k < NB; ++k) ok = ok && (bnd[k] > bnd[k - 1]);
      if (!ok) par[0] = 1u;
    }
    __syncthreads();
    for (int c = threadIdx.x; c < EM_CELLS; c += EM_THREADS) {
      uint32_t base = 0, cnt = 0;
      float inside = INFINITY;
      for (int k = 0; k < NB; ++k) {
        const uint32_t cb = em_cell(bnd[k]) >> 3;
        if (cb < (uint32_t)c) ++base;
        if (cb == (uint32_t)c) { ++cnt; inside = bnd[k]; }
      }
      uint32_t* lut = (uint32_t*)(lds + EM_LUT_OFF);
      lut[2 * c] = base;
      lut[2 * c + 1] = __float_as_uint(inside);
      if (cnt > 1) atomicOr(par, 1u);
    }
    __syncthreads();
  };
  const float* bnd = (const float*)(lds + EM_BND_OFF);

  unsigned char* wl = lds + WAVE_OFF + wave * EM_WAVE_BYTES;
  int64_t* src_off = (int64_t*)wl;                    // address of the vector, or 0
  int64_t* dst_p = (int64_t*)(wl + ROWS * 8);      // address of the packed row, or 0
  int64_t* dst_n = (int64_t*)(wl + ROWS * 16);     // address of the norm
  float* rinv = (float*)(wl + ROWS * 24);          // 1/(|x| + 1e-10), scaled back by 1/EM_PSCALE; NaN rows flagged

  const int64_t n_total = (PAGED && a.x2) ? 2 * a.n : a.n;      // a second tensor rides along (K and V of a step)
  const int64_t steps = (n_total + ROWS - 1) / ROWS;
  const int64_t stride = SPLIT ? (int64_t)gridDim.x : (int64_t)gridDim.x * EM_WAVES;
  // SPLIT: the wavefront's N-tile of the B operand, both terms, four k-steps
  em_half8 Bh[4], Bl[4];
  if constexpr (SPLIT) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      union { uint4 u; em_half8 h; } ch, cl;
      ch.u = bop[(wave * 4 + ks) * 64 + lane];
      cl.u = bop[2048 + (wave * 4 + ks) * 64 + lane];
      Bh[ks] = ch.h;
      Bl[ks] = cl.h;
    }
  }

  // A operands of one step straight from memory (zeros past the end): lane l resolves the source
  // row of vector base + l, the lanes of an M-tile pick the rows up through LDS
  // (a row's 32 elements of the lane as 16-byte pieces: four for 16-bit input -- the A operands themselves --
  // eight for float32 input)
  constexpr int NP = 4 * NA;
  auto fetch = [&](uint4 (&R)[MT][NP], int64_t step) {
    if constexpr (DIRECT) {
      // contiguous rows whose byte offsets fit 31 bits: every lane forms its rows' addresses itself
      // (scalar base + 32-bit lane offset), no exchange through LDS
      if ((uint32_t)step * ROWS + ROWS <= (uint32_t)a.n) {      // a whole step (all but the last): nothing to check
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const uint32_t n = (uint32_t)step * ROWS + 16 * mt + (lane & 15);
          const uint4* p = (const uint4*)((const char*)a.x + (n * (uint32_t)a.xs0 + 32u * g) * (uint32_t)XB);
#pragma unroll
          for (int ks = 0; ks < NP; ++ks) R[mt][ks] = p[ks];
        }
        return;
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const uint32_t n = (uint32_t)step * ROWS + 16 * mt + (lane & 15);
        if (n < (uint32_t)a.n) {
          const uint4* p = (const uint4*)((const char*)a.x + (n * (uint32_t)a.xs0 + 32u * g) * (uint32_t)XB);
#pragma unroll
          for (int ks = 0; ks < NP; ++ks) R[mt][ks] = p[ks];
        } else {
#pragma unroll
          for (int ks = 0; ks < NP; ++ks) R[mt][ks] = make_uint4(0u, 0u, 0u, 0u);
        }
      }
      return;
    }
    int64_t n = step * ROWS + lane;
    int64_t so = 0;      // byte address of the vector, 0 = none
    if (step < steps && n < n_total && lane < ROWS) {
      const bool second = PAGED && n >= a.n;
      if (second) n -= a.n;
      const char* xb = (const char*)(second ? a.x2 : a.x);
      if (PAGED) {
        const int64_t tok = n / a.heads, head = n - tok * a.heads;
        so = (int64_t)(uintptr_t)(xb + XB * (tok * a.xs0 + head * a.xs1));
      } else {
        so = (int64_t)(uintptr_t)(xb + XB * n * a.xs0);
      }
    }
    if (lane < ROWS) src_off[lane] = so;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int64_t ro = src_off[16 * mt + (lane & 15)];
      if (ro != 0) {
        const uint4* p = (const uint4*)(uintptr_t)(ro + 32 * XB * g);
#pragma unroll
        for (int ks = 0; ks < NP; ++ks) R[mt][ks] = p[ks];
      } else {
#pragma unroll
        for (int ks = 0; ks < NP; ++ks) R[mt][ks] = make_uint4(0u, 0u, 0u, 0u);
      }
    }
  };

  auto encode_step = [&](auto linear_tag, int64_t step, uint4 (&R)[MT][NP]) {
    constexpr bool LINEAR = decltype(linear_tag)::value;
    em_half8 A[MT][4];          // the operand (16-bit input), or its float16 hi term (float32 input)
    em_half8 Alo[MT][4];        // float32 input: the lo term
    if constexpr (XDT != AKV_F32) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          union { uint4 u; em_half8 h; } cv;
          cv.u = R[mt][ks];
          A[mt][ks] = cv.h;
        }
    }
    const int64_t base = step * ROWS;
    // ---- lane l resolves the destination of vector base + l
    if constexpr (!DIRECT) {
      int64_t n = base + lane;
      int64_t dp = 0, dn = 0;      // byte addresses of the packed row and of the norm, 0 = skip
      if (n < n_total && lane < ROWS) {
        const bool second = PAGED && n >= a.n;
        if (second) n -= a.n;
        uint8_t* pb = second ? a.packed2 : a.packed;
        float* nb = second ? a.norms2 : a.norms;
        if (PAGED) {
          const int64_t tok = n / a.heads, head = n - tok * a.heads;
          const int64_t slot = akv_load_index(a.slots, a.slot_itype, tok);
          if (slot >= 0) {
            const int64_t blk = slot / a.block_size, pos = slot - blk * a.block_size;
            if (blk < a.max_blocks) {
              dp = (int64_t)(uintptr_t)(pb + blk * a.ps0 + pos * a.ps1 + head * a.ps2);
              dn = (int64_t)(uintptr_t)(nb + blk * a.ns0 + pos * a.ns1 + head * a.ns2);
            }
          }
        } else {
          dp = (int64_t)(uintptr_t)(pb + n * a.ps0);
          dn = (int64_t)(uintptr_t)(nb + n);
        }
      }
      if (lane < ROWS) {
        dst_p[lane] = dp;
        dst_n[lane] = dn;
      }
    }
    float ss[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) ss[mt] = 0.f;
    uint32_t unscale[MT];     // float bits of the power of two taken out of each M-tile's rows
    bool nonfinite[MT];       // bfloat16 only: the row holds an infinity or a NaN
    if constexpr (XDT == AKV_F16) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        unscale[mt] = 0x3f800000u;
        nonfinite[mt] = false;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          union { em_half8 h; em_half2 h2[4]; } cv;
          cv.h = A[mt][ks];
#pragma unroll
          for (int q = 0; q < 4; ++q) ss[mt] = __builtin_amdgcn_fdot2(cv.h2[q], cv.h2[q], ss[mt], false);
        }
      }
    } else if constexpr (XDT == AKV_F32) {
      // float32 rows: squared norm from the values themselves; then each row is scaled by the power of two
      // that brings its largest element into [1, 2) and split into two float16 terms, both rounded to
      // nearest: hi keeps 11 bits, x - hi is exact in float32 and has at most 12 significant bits and a sign,
      // so lo is off by at most half a float32 ulp of the element (2^-25 of the largest element once lo is a
      // float16 subnormal)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        uint32_t mx = 0u;
#pragma unroll
        for (int pc = 0; pc < NP; ++pc) {
          const uint32_t w[4] = {R[mt][pc].x, R[mt][pc].y, R[mt][pc].z, R[mt][pc].w};
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            mx = max(mx, w[q] & 0x7fffffffu);
            const float v = __uint_as_float(w[q]);
            ss[mt] = fmaf(v, v, ss[mt]);
          }
        }
        {   // largest magnitude of the row over its four lanes
          auto r1 = __builtin_amdgcn_permlane32_swap(mx, mx, false, false);
          mx = max(r1[0], r1[1]);
          auto r2 = __builtin_amdgcn_permlane16_swap(mx, mx, false, false);
          mx = max(r2[0], r2[1]);
        }
        uint32_t ef = mx >> 23;                      // exponent field of the largest element
        nonfinite[mt] = ef == 255u;
        if (ef == 0u || ef == 255u) ef = 127u;       // all (sub)zero, or not finite (flagged)
        if (ef == 254u) ef = 253u;                   // keep the scale a normal number
        const float sc = __uint_as_float((254u - ef) << 23);     // 2^(127 - ef)
        unscale[mt] = ef << 23;                                   // 2^(ef - 127)
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const float v[8] = {__uint_as_float(R[mt][2 * ks].x), __uint_as_float(R[mt][2 * ks].y),
                              __uint_as_float(R[mt][2 * ks].z), __uint_as_float(R[mt][2 * ks].w),
                              __uint_as_float(R[mt][2 * ks + 1].x), __uint_as_float(R[mt][2 * ks + 1].y),
                              __uint_as_float(R[mt][2 * ks + 1].z), __uint_as_float(R[mt][2 * ks + 1].w)};
          union { em_half8 h; em_half2 h2[4]; } hi, lo;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float x0 = v[2 * q] * sc, x1 = v[2 * q + 1] * sc;
            const _Float16 h0 = (_Float16)x0, h1 = (_Float16)x1;
            hi.h2[q] = (em_half2){h0, h1};
            lo.h2[q] = (em_half2){(_Float16)(x0 - (float)h0), (_Float16)(x1 - (float)h1)};
          }
          A[mt][ks] = hi.h;
          Alo[mt][ks] = lo.h;
        }
      }
    } else {
      // bfloat16 rows: squared norm from the exact float32 values; then each row is scaled by the
      // power of two that brings its largest element into [1, 2) and converted to float16 -- exact
      // for every element within 2^14 of the largest (8 significant bits fit in 11), and off by at
      // most 2^-25 of the largest otherwise, far below the resolution of the codebook search
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        em_us2 mx2 = {0, 0};
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          union { em_half8 h; uint32_t w[4]; } cv;
          cv.h = A[mt][ks];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            union { uint32_t u; em_us2 v; } mm;
            mm.u = cv.w[q] & 0x7fff7fffu;
            mx2 = __builtin_elementwise_max(mx2, mm.v);
            const float lo = __uint_as_float(cv.w[q] << 16), hi = __uint_as_float(cv.w[q] & 0xffff0000u);
            ss[mt] = fmaf(lo, lo, ss[mt]);
            ss[mt] = fmaf(hi, hi, ss[mt]);
          }
        }
        uint32_t mx = max((uint32_t)mx2[0], (uint32_t)mx2[1]);
        {   // largest magnitude of the row over its four lanes
          auto r1 = __builtin_amdgcn_permlane32_swap(mx, mx, false, false);
          mx = max(r1[0], r1[1]);
          auto r2 = __builtin_amdgcn_permlane16_swap(mx, mx, false, false);
          mx = max(r2[0], r2[1]);
        }
        uint32_t ef = mx >> 7;                       // exponent field of the largest element
        nonfinite[mt] = ef == 255u;
        if (ef == 0u || ef == 255u) ef = 127u;       // all (sub)zero, or not finite (flagged)
        if (ef == 254u) ef = 253u;                   // keep the scale a normal number
        const float sc = __uint_as_float((254u - ef) << 23);     // 2^(127 - ef)
        unscale[mt] = ef << 23;                                   // 2^(ef - 127)
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          union { em_half8 h; uint32_t w[4]; em_half2 h2[4]; } cv;
          cv.h = A[mt][ks];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float lo = __uint_as_float(cv.w[q] << 16) * sc, hi = __uint_as_float(cv.w[q] & 0xffff0000u) * sc;
            auto pk = __builtin_amdgcn_cvt_pkrtz(lo, hi);
            cv.h2[q] = (em_half2){(_Float16)pk[0], (_Float16)pk[1]};
          }
          A[mt][ks] = cv.h;
        }
      }
    }
    // lane l < ROWS finishes vector l = 16 mt + row: transpose-reduce the partial sums over the
    // four lanes of a row
    bool any_nan;       // some vector of the step holds a NaN or an infinity (the same in every lane)
    {
      const bool g1 = (g & 1) != 0;
      float mine;
      if constexpr (MT == 1) {
        const float a01 = ss[0] + akv_lane_xor<16>(ss[0]);     // (row swaps, not shuffles: the step waits for this chain)
        mine = a01 + akv_lane_xor<32>(a01);                   // all four lanes of a row hold its sum
      } else {
        static_assert(MT <= 2, "two M-tiles at most");
        const float a01 = (g1 ? ss[MT - 1] : ss[0]) + akv_lane_xor<16>(g1 ? ss[0] : ss[MT - 1]);
        mine = a01 + akv_lane_xor<32>(a01);                   // lanes g and g + 2 both hold M-tile g & 1
      }
      const float nrm = sqrtf(mine);
      const uint32_t my_unscale = (MT > 1 && g1) ? unscale[MT - 1] : unscale[0];
      const float r = (1.f / (nrm + 1e-10f)) * (1.f / EM_PSCALE) * __uint_as_float(my_unscale);
      // a vector with a NaN or an infinity rotates to NaN everywhere: every code is the last level.
      // (float16 squares cannot overflow, so there an infinite norm means an infinite element; a
      // finite bfloat16 row whose squares overflow has norm inf, unit vector 0 and y = 0 like the
      // reference: r is 0 and the scaled products are finite.)
      const bool my_nonfinite = (MT > 1 && g1) ? nonfinite[MT - 1] : nonfinite[0];
      const bool nan_row = XDT == AKV_F16 ? !(nrm < INFINITY) : (my_nonfinite || nrm != nrm);   // (float32 as bfloat16)
      any_nan = __ballot(nan_row && lane < ROWS) != 0;
      if (lane < ROWS) {
        rinv[lane] = nan_row ? __uint_as_float(0x7fc00000u) : r;
        if constexpr (DIRECT) {
          if ((uint32_t)base + lane < (uint32_t)a.n) a.norms[(uint32_t)base + lane] = nrm;
        } else {
          if (dst_p[lane] != 0 && (!SPLIT || wave == 0)) *(float*)(uintptr_t)dst_n[lane] = nrm;
        }
      }
    }
    if constexpr (SPLIT) {
      // ---- the wavefront's tile: products, reciprocal, comparison with every boundary, code bytes to LDS
      union { em_u32x4 u; em_float4 f; } rc;
      rc.u = *(em_lds_u128*)(uintptr_t)(uint32_t)(WAVE_OFF + wave * EM_WAVE_BYTES + ROWS * 24 + (4 * g) * 4);
      em_float4 acc = (em_float4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[0][ks], Bh[ks], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[0][ks], Bl[ks], acc, 0, 0, 0);
      }
      uint8_t* codes = lds + EM_SPLIT_CODES;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float y = acc[i] * rc.f[i];
        uint32_t code = 0;
#pragma unroll
        for (int k = 0; k < NB; ++k) code += (a.table[k] < y) ? 1u : 0u;
        if (!(rc.f[i] == rc.f[i])) code = (uint32_t)NB;            // NaN vector: last level everywhere
        codes[(4 * g + i) * 128 + 8 * col + wave] = (uint8_t)code;
      }
      __syncthreads();
      if (threadIdx.x < 256) {
        const int row = threadIdx.x >> 4, grp = threadIdx.x & 15;
        const int64_t dp = dst_p[row];
        if (dp != 0) {
          const uint2 c8 = *(const uint2*)(codes + row * 128 + 8 * grp);
          auto code_of = [&](int t) { return ((t < 4 ? c8.x : c8.y) >> (8 * (t & 3))) & 0xffu; };
          uint32_t v = 0;
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            const int t = BITS == 4 ? 6 - (k & ~1) + (k & 1) : BITS == 3 ? k : ((k + 4) & 7);
            v = (v << BITS) + code_of(t);
          }
          uint8_t* prow = (uint8_t*)(uintptr_t)dp;
          if (BITS == 4) {
            *(uint32_t*)(prow + 4 * grp) = v;
          } else if (BITS == 3) {
            prow[3 * grp] = (uint8_t)(v >> 16);
            prow[3 * grp + 1] = (uint8_t)(v >> 8);
            prow[3 * grp + 2] = (uint8_t)v;
          } else {
            *(uint16_t*)(prow + 2 * grp) = (uint16_t)v;
          }
        }
      }
      __syncthreads();      // the code bytes are rewritten by the next step
      return;
    }
    // ---- rotate, search, pack
    uint32_t packed[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) packed[mt][i] = 0u;
    em_float4 rv[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      union { em_u32x4 u; em_float4 f; } cv;
      cv.u = *(em_lds_u128*)(uintptr_t)(uint32_t)(WAVE_OFF + wave * EM_WAVE_BYTES + ROWS * 24 + (16 * mt + 4 * g) * 4);
      rv[mt] = cv.f;
    }
    // N-tiles are software-pipelined: the matrix-core work of tile nt + 1 is issued together with
    // the search of tile nt (independent instruction streams in one basic block), so the vector
    // unit works in the shadow of the MFMAs.  The loop stays rolled (two tiles per pass): unrolled,
    // the scheduler would want every B operand in registers at once.
    auto mfma_tile = [&](int nt, em_float4 (&acc)[MT]) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = (em_float4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        union { em_u32x4 u; em_half8 h; } bh, bl;
        bh.u = *(em_lds_u128*)(uintptr_t)(uint32_t)(EM_B_OFF + ((nt * 4 + ks) * 64 + lane) * 16);
        bl.u = *(em_lds_u128*)(uintptr_t)(uint32_t)(EM_B_OFF + 32768 + ((nt * 4 + ks) * 64 + lane) * 16);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[mt][ks], bh.h, acc[mt], 0, 0, 0);
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[mt][ks], bl.h, acc[mt], 0, 0, 0);
          if constexpr (XDT == AKV_F32)
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Alo[mt][ks], bh.h, acc[mt], 0, 0, 0);
        }
      }
    };
    // A lane's packed group is built by shift-and-add, one instruction per code: the N-tiles are visited
    // in the order in which their codes enter the group from the top (4-bit: 6 7 4 5 2 3 0 1 -- a dword
    // is four little-endian bytes of two nibbles; 3-bit: 0 .. 7; 2-bit: 4 5 6 7 0 1 2 3).
    auto tile_at = [&](int k) -> int {
      return BITS == 4 ? 6 - (k & ~1) + (k & 1) : BITS == 3 ? k : ((k + 4) & 7);
    };
    auto search_tile = [&](const em_float4 (&acc)[MT]) {
      float y[MT][4];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) y[mt][i] = acc[mt][i] * rv[mt][i];
      if constexpr (!LINEAR) {
        em_u32x2 e[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            e[mt][i] = *(em_lds_u64*)(uintptr_t)em_cell(y[mt][i]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t code = e[mt][i].x + ((__uint_as_float(e[mt][i].y) < y[mt][i]) ? 1u : 0u);
            packed[mt][i] = (packed[mt][i] << BITS) + code;
          }
      } else {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            uint32_t code = 0;
#pragma unroll 1
            for (int k = 0; k < NB; ++k) code += (bnd[k] < y[mt][i]) ? 1u : 0u;
            packed[mt][i] = (packed[mt][i] << BITS) + code;
          }
      }
    };
    em_float4 accA[MT], accB[MT];
    mfma_tile(tile_at(0), accA);
#pragma unroll 1
    for (int k = 0; k < 6; k += 2) {
      mfma_tile(tile_at(k + 1), accB);
      search_tile(accA);
      mfma_tile(tile_at(k + 2), accA);
      search_tile(accB);
      // issue order of the pass: one MFMA, then the vector and LDS work that fits in its shadow
#pragma unroll
      for (int q = 0; q < 8 * (NA + 1) * MT; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);   // VALU
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // LDS read
      }
    }
    mfma_tile(tile_at(7), accB);
    search_tile(accA);
#pragma unroll
    for (int q = 0; q < 4 * (NA + 1) * MT; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    search_tile(accB);
    // ---- store: lane (col, g) writes group col of rows 4g + i
    auto put = [&](uint8_t* prow, uint32_t v) {
      if (BITS == 4) {
        *(uint32_t*)(prow + 4 * col) = v;
      } else if (BITS == 3) {
        prow[3 * col] = (uint8_t)(v >> 16);
        prow[3 * col + 1] = (uint8_t)(v >> 8);
        prow[3 * col + 2] = (uint8_t)v;
      } else {
        *(uint16_t*)(prow + 2 * col) = (uint16_t)v;
      }
    };
    if (DIRECT && !any_nan && (uint32_t)base + ROWS <= (uint32_t)a.n) {
      // a whole step of finite vectors (all but a few): the row's address is a scalar (step and row number)
      // plus the lane's own offset (its row quarter and group), nothing is checked
      const uint32_t lane_off = (uint32_t)(4 * g) * (uint32_t)a.ps0;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          put(a.packed + (uint64_t)((uint32_t)base + 16 * mt + i) * (uint32_t)a.ps0 + lane_off, packed[mt][i]);
      return;
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = 16 * mt + 4 * g + i;
        uint8_t* prow;
        if constexpr (DIRECT) {
          const uint32_t n = (uint32_t)base + row;
          if (n >= (uint32_t)a.n) continue;
          prow = a.packed + n * (uint32_t)a.ps0;
        } else {
          const int64_t dp = dst_p[row];
          if (dp == 0) continue;
          prow = (uint8_t*)(uintptr_t)dp;
        }
        uint32_t v = packed[mt][i];
        if (!(rv[mt][i] == rv[mt][i])) v = 0xffffffffu;     // NaN vector: last level everywhere
        put(prow, v);
      }
  };

  // the rows of a step are requested at the end of the step before it (the first: before the set-up)
  const int64_t first = SPLIT ? (int64_t)blockIdx.x : (int64_t)wave * gridDim.x + blockIdx.x;
  uint4 R[MT][NP];
  fetch(R, first);
  if constexpr (SPLIT) {
    for (int64_t step = first; step < steps; step += stride) {      // (the same steps in every wavefront)
      encode_step(std::true_type{}, step, R);
      fetch(R, step + stride);
    }
    return;
  }
  setup();
  const bool linear_search = ((const uint32_t*)(lds + EM_PAR_OFF))[0] != 0;   // uniform
  if (__builtin_expect(!linear_search, 1)) {
    for (int64_t step = first; step < steps; step += stride) {
      encode_step(std::false_type{}, step, R);
      fetch(R, step + stride);
    }
  } else {
    for (int64_t step = first; step < steps; step += stride) {
      encode_step(std::true_type{}, step, R);
      fetch(R, step + stride);
    }
  }
}

// the split form exists for 16-bit rows addressed row by row; returns false where it does not
template <int BB, bool PG, int DT, bool DR>
static bool em_launch_split(int grid, hipStream_t stream, const akv_gen_args& a, const uint4* bop) {
  if constexpr (DT != AKV_F32 && !DR) {
    AKV_LAUNCH_TIMED((akv_encode_mfma_kernel<BB, PG, DT, false, 1, true>), grid, EM_SPLIT_WAVES * 64, EM_SPLIT_LDS_BYTES,
                     stream, a, bop);
    return true;
  } else {
    return false;
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
  if (em_disabled() || d != 128 || (x_dtype != AKV_F16 && x_dtype != AKV_BF16 && x_dtype != AKV_F32)) return AKV_ERR_UNSUPPORTED;
  // 16-byte loads of the input rows; aligned stores of the packed groups
  const int64_t xmask = x_dtype == AKV_F32 ? 3 : 7;        // elements per 16 bytes, minus one
  if (((uintptr_t)a.x & 15) || ((uintptr_t)a.x2 & 15) || (a.xs0 & xmask) || (paged && (a.xs1 & xmask))) return AKV_ERR_UNSUPPORTED;
  const int64_t amask = bits == 4 ? 3 : bits == 2 ? 1 : 0;
  if (((uintptr_t)a.packed | (uintptr_t)a.packed2 | (uintptr_t)a.ps0 | (uintptr_t)a.ps1 | (uintptr_t)a.ps2) & amask) return AKV_ERR_UNSUPPORTED;
  const uint4* bop = (const uint4*)((const float*)rot_prep + (size_t)2 * d * d);
  const int64_t n_total = (paged && a.x2) ? 2 * a.n : a.n;
  const int cus = akv_cached_cu_count();
  // A call too small to give every CU a step of 32 vectors (one serving step: 4,096 vectors) runs the form with 16
  // vectors per wavefront step: twice the workgroups, half the chain of products and searches that its one busy
  // wavefront per workgroup walks through alone.
  const bool narrow = paged && x_dtype != AKV_F32 && (n_total + EM_ROWS - 1) / EM_ROWS < cus;
  // ... and one (paged or flat) that leaves a workgroup at most two steps of 16 vectors shares each step among
  // eight wavefronts
  const bool split = x_dtype != AKV_F32 && (n_total + 15) / 16 <= 2 * (int64_t)cus && !getenv("AKV_ENCODE_NO_SPLIT");
  const int rows_per_step = (x_dtype == AKV_F32 || narrow || split) ? 16 : EM_ROWS;
  const int64_t steps = (n_total + rows_per_step - 1) / rows_per_step;
  // steps are dealt round-robin over workgroups first, so a small call (one serving step) spreads
  // over as many CUs as it has steps instead of filling the wavefronts of a few
  const int grid = (int)(steps < cus ? steps : cus);
#define EM_LAUNCH_MT(BB, PG, DT, DR, MM)                                                              \
  do {                                                                                               \
    static bool configured = false;                                                                  \
    if (!configured) {                                                                               \
      AKV_HIP(hipFuncSetAttribute((const void*)akv_encode_mfma_kernel<BB, PG, DT, DR, MM>,            \
                                  hipFuncAttributeMaxDynamicSharedMemorySize, EM_LDS_BYTES));        \
      configured = true;                                                                             \
    }                                                                                                \
    AKV_LAUNCH_TIMED((akv_encode_mfma_kernel<BB, PG, DT, DR, MM>), grid, EM_THREADS, EM_LDS_BYTES, stream, a, bop); \
  } while (0)
#define EM_LAUNCH(BB, PG, DT, DR)                                                                     \
  do {                                                                                               \
    if (split && em_launch_split<BB, PG, DT, DR>(grid, stream, a, bop)) break;                       \
    if (DT == AKV_F32 || (PG && narrow)) EM_LAUNCH_MT(BB, PG, DT, DR, 1);                             \
    else EM_LAUNCH_MT(BB, PG, DT, DR, (DT == AKV_F32 ? 1 : EM_MT));                                   \
  } while (0)
#define EM_LAUNCH_DT(BB, PG, DR) do { if (x_dtype == AKV_F16) EM_LAUNCH(BB, PG, AKV_F16, DR); else if (x_dtype == AKV_BF16) EM_LAUNCH(BB, PG, AKV_BF16, DR); else EM_LAUNCH(BB, PG, AKV_F32, DR); } while (0)
  // flat rows whose byte offsets stay below 2^31 take the variant with 32-bit lane offsets
  const int64_t xbytes = x_dtype == AKV_F32 ? 4 : 2;
  const bool direct = !paged && a.n < ((int64_t)1 << 31) / (xbytes * a.xs0 > a.ps0 ? xbytes * a.xs0 : a.ps0);
  if (paged) {
    if (bits == 4) EM_LAUNCH_DT(4, true, false); else if (bits == 3) EM_LAUNCH_DT(3, true, false); else EM_LAUNCH_DT(2, true, false);
  } else if (direct && !split) {
    if (bits == 4) EM_LAUNCH_DT(4, false, true); else if (bits == 3) EM_LAUNCH_DT(3, false, true); else EM_LAUNCH_DT(2, false, true);
  } else {
    if (bits == 4) EM_LAUNCH_DT(4, false, false); else if (bits == 3) EM_LAUNCH_DT(3, false, false); else EM_LAUNCH_DT(2, false, false);
  }
#undef EM_LAUNCH_DT
#undef EM_LAUNCH
#undef EM_LAUNCH_MT
  AKV_LAUNCH_CHECK("akv_encode_mfma_kernel");
  return AKV_OK;
}
