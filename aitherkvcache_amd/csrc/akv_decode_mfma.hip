// MFMA decode (unpack -> centroid lookup -> inverse rotation -> x norm -> cast) for the 4-, 3- and
// 2-bit codecs at head_dim 128: TurboQuant.decode, aither_kvcache/quantizer.py:168-197.
//
//   X[v, i] = n_v * sum_j c[code[v, j]] * Pi[j, i]              v_mfma_f32_16x16x32_f16
//     A = centroids of the codes: lane (row = l%16, g = l/16) loads bytes [16g, 16g+16) of the
//         vector's packed row (one 16-byte load) = coordinates j = 32g .. 32g+31; k-step ks takes
//         dword ks of them.  A code BYTE (two codes) indexes a table in LDS whose entry is the
//         float16 pair (c[a], c[b]); the table has a hi and a lo half (c = hi + lo to ~22 bits)
//         and every entry is replicated 32 times (address = byte * 256 + (lane & 31) * 4, built
//         by one byte permute) so lookups never conflict on a bank.
//     B = Pi split into two float16 terms (hi + lo, scaled by 64).  Three MFMAs per tile:
//         c_hi Pi_hi + c_lo Pi_hi + c_hi Pi_lo.  N-tile nt, column col is output element
//         i = 8 col + nt, so that over the eight N-tiles a lane collects eight consecutive
//         elements of a row: one 16-byte store, sixteen lanes write the 256-byte row.
//     k-steps are the outer loop (A operands of one k-step live in registers, all 8 x 2
//     accumulator tiles stay resident).
//
// 3-bit and 2-bit rows are spread to one code per nibble in registers (akv_nibble.h) and then take the
// same table and products; the coordinate order that the spreading leaves is matched by the order in
// which the rows of the B operand are copied into LDS.
//
// A wavefront decodes 32 vectors per step; a workgroup is eight independent wavefronts plus the
// B operand (64 KB) and the byte table (64 KB).
#include "akv_common.h"
#include "akv_nibble.h"

typedef _Float16 dm_half8 __attribute__((ext_vector_type(8)));
typedef float dm_float4 __attribute__((ext_vector_type(4)));
typedef uint32_t dm_u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) dm_u32x4 dm_lds_u128;
typedef __attribute__((address_space(3))) const uint32_t dm_lds_cu32;

#define DM_WAVES 8
#define DM_THREADS (DM_WAVES * 64)
#define DM_ROWS 32
#define DM_PSCALE 64.f
#define DM_LUT_OFF 0                 // 256 entries x 256 B: [hi pair x 32 copies][lo pair x 32 copies]
#define DM_B_OFF 65536               // [hi/lo][8 nt][4 ks][64 lanes] x 16 B
#define DM_ROW_OFF 131072            // per wavefront: DM_ROWS x {packed offset, norm offset, output offset} (block-wise decode)
#define DM_LDS_BYTES (131072 + DM_WAVES * DM_ROWS * 24)
#define DM_SEL(k) (0x0c0c0400u + ((uint32_t)(k) << 8))

// the lane's quarter of a packed row: 16 / 12 / 8 bytes
template <int BITS>
__device__ __forceinline__ uint4 dm_load_quarter(const uint8_t* row, int g) {
  if constexpr (BITS == 4) {
    return *(const uint4*)(row + 16 * g);
  } else if constexpr (BITS == 3) {
    const uint32_t* p = (const uint32_t*)(row + 12 * g);
    return make_uint4(p[0], p[1], p[2], 0u);
  } else {
    const uint2 t = *(const uint2*)(row + 8 * g);
    return make_uint4(t.x, t.y, 0u, 0u);
  }
}

// B operand of the decode kernel, stored after the encode operand in the prepared-rotation buffer
__global__ __launch_bounds__(256) void akv_dm_prepare_kernel(const float* __restrict__ Pi, uint4* __restrict__ bop) {
  const int t = blockIdx.x * 256 + threadIdx.x;      // (nt, ks, lane): 2048 threads
  const int lane = t & 63, ks = (t >> 6) & 3, nt = t >> 8;
  const int col = lane & 15, g = lane >> 4;
  const int i = 8 * col + nt;
  uint32_t hi[4], lo[4];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float v = Pi[(size_t)(32 * g + 8 * ks + e) * 128 + i] * DM_PSCALE;
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

int akv_prepare_decode_mfma(const float* rotation, int d, void* prep, hipStream_t stream) {
  if (d != 128) return AKV_OK;
  uint4* bop = (uint4*)((char*)prep + AKV_PREP_DECODE_OFFSET(d));
  akv_dm_prepare_kernel<<<8, 256, 0, stream>>>(rotation, bop);
  AKV_LAUNCH_CHECK("akv_dm_prepare_kernel");
  return AKV_OK;
}

// BLOCKS = false: n contiguous rows (TurboQuant.decode).  BLOCKS = true: the rows are the
// (position, head) entries of the cache blocks listed in a.slots; every listed block that exists is
// decoded into the block of the same index of the output buffer (the batch decompress of
// aither_kvcache/vllm/backend.py:1040-1091 without its gather / unique / scatter passes).
template <bool BLOCKS, int BITS, int ODT>
__global__ __launch_bounds__(DM_THREADS) void akv_decode_mfma_kernel(akv_gen_args a, const uint4* __restrict__ bop) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 15, g = lane >> 4;
  {
    if constexpr (BITS == 4) {
      uint4* b_lds = (uint4*)(lds + DM_B_OFF);
      for (int i = threadIdx.x; i < 65536 / 16; i += DM_THREADS) b_lds[i] = bop[i];
    } else {
      // element e of k-step ks of a lane faces the coordinate that the spread code stream holds there
      const uint16_t* src = (const uint16_t*)bop;
      uint16_t* b_lds = (uint16_t*)(lds + DM_B_OFF);
      for (int i = threadIdx.x; i < 65536 / 2; i += DM_THREADS) {
        const int e = i & 7, ln = (i >> 3) & 63, ks = (i >> 9) & 3, rest = i >> 11;   // rest = (hi | lo, nt)
        const int c = mf_kcoord<BITS>(ks, e >> 1, e & 1);
        b_lds[i] = src[((rest * 4 + (c >> 3)) * 64 + ln) * 8 + (c & 7)];
      }
    }
    // byte table: entry (hi nibble, lo nibble) -> (c[hi nibble], c[lo nibble]): the code of the
    // even coordinate is the high nibble (packing.py:13-23) and goes to the low half of the pair
    uint32_t* lut = (uint32_t*)(lds + DM_LUT_OFF);
    for (int i = threadIdx.x; i < 256 * 64; i += DM_THREADS) {
      const int e = i >> 6, half = (i >> 5) & 1;
      constexpr int LM = (1 << BITS) - 1;      // nibble values above the top level do not occur
      const float c0 = a.table[(e >> 4) & LM], c1 = a.table[e & 15 & LM];
      const __half h0 = __float2half_rn(c0), h1 = __float2half_rn(c1);
      uint32_t w;
      if (half == 0) {
        w = (uint32_t)__half_as_ushort(h0) | ((uint32_t)__half_as_ushort(h1) << 16);
      } else {
        const __half l0 = __float2half_rn(c0 - __half2float(h0)), l1 = __float2half_rn(c1 - __half2float(h1));
        w = (uint32_t)__half_as_ushort(l0) | ((uint32_t)__half_as_ushort(l1) << 16);
      }
      lut[i] = w;
    }
    __syncthreads();
  }
  const uint32_t lane4 = (uint32_t)(lane & 31) * 4u;
  const uint32_t b_addr = DM_B_OFF + (uint32_t)lane * 16u;

  const int64_t steps = (a.n + DM_ROWS - 1) / DM_ROWS;
  const int64_t stride = (int64_t)gridDim.x * DM_WAVES;
  for (int64_t step = (int64_t)wave * gridDim.x + blockIdx.x; step < steps; step += stride) {
    const int64_t base = step * DM_ROWS;
    // ---- packed rows and norms
    uint4 pk[2];
    float4 nr[2];
    int64_t* row_p = (int64_t*)(lds + DM_ROW_OFF + wave * DM_ROWS * 24);   // packed byte offset, or -1
    int64_t* row_n = row_p + DM_ROWS;                                      // norm element offset
    int64_t* row_o = row_n + DM_ROWS;                                      // output element offset
    if constexpr (BLOCKS) {
      if (lane < DM_ROWS) {   // lane l resolves row base + l = (listed block, position, head)
        const int64_t n = base + lane;
        int64_t po = -1, no = 0, oo = 0;
        if (n < a.n) {
          const int64_t per_blk = (int64_t)a.block_size * a.heads;
          const int64_t li = n / per_blk, rem = n - li * per_blk;
          const int64_t pos = rem / a.heads, head = rem - pos * a.heads;
          const int64_t blk = akv_load_index(a.slots, a.slot_itype, li);
          if (blk >= 0 && blk < a.max_blocks) {
            po = blk * a.ps0 + pos * a.ps1 + head * a.ps2;
            no = blk * a.ns0 + pos * a.ns1 + head * a.ns2;
            oo = blk * a.os0 + pos * a.os1 + head * a.os2;
          }
        }
        row_p[lane] = po; row_n[lane] = no; row_o[lane] = oo;
      }
    }
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      float nv[4];
      if constexpr (BLOCKS) {
        const int64_t po = row_p[16 * mt + (lane & 15)];
        pk[mt] = po >= 0 ? dm_load_quarter<BITS>(a.packed + po, g) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 16 * mt + 4 * g + i;
          nv[i] = row_p[r] >= 0 ? a.norms[row_n[r]] : 0.f;
        }
      } else {
        const int64_t n = base + 16 * mt + (lane & 15);
        pk[mt] = n < a.n ? dm_load_quarter<BITS>(a.packed + n * a.ps0, g) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int64_t r = base + 16 * mt + 4 * g + i;
          nv[i] = r < a.n ? a.norms[r] : 0.f;
        }
      }
      nr[mt] = make_float4(nv[0], nv[1], nv[2], nv[3]);
    }
    uint32_t kw[2][4];      // one code per nibble
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      const uint32_t raw[4] = {pk[mt].x, pk[mt].y, pk[mt].z, pk[mt].w};
      mf_spread_row<BITS>(raw, kw[mt]);
    }
    dm_float4 acc[2][8];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nt = 0; nt < 8; ++nt) acc[mt][nt] = (dm_float4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      // A operands of this k-step: four byte lookups (hi and lo) per M-tile
      dm_half8 ah[2], al[2];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const uint32_t w = kw[mt][ks];
        union { uint32_t u[4]; dm_half8 h; } ch, cl;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const uint32_t addr = __builtin_amdgcn_perm(w, lane4, DM_SEL(b));
          ch.u[b] = *(dm_lds_cu32*)(uintptr_t)addr;
          cl.u[b] = *(dm_lds_cu32*)(uintptr_t)(addr + 128u);
        }
        ah[mt] = ch.h;
        al[mt] = cl.h;
      }
#pragma unroll
      for (int nt = 0; nt < 8; ++nt) {
        union { dm_u32x4 u; dm_half8 h; } bh, bl;
        bh.u = *(dm_lds_u128*)(uintptr_t)(b_addr + (uint32_t)((nt * 4 + ks) * 1024));
        bl.u = *(dm_lds_u128*)(uintptr_t)(b_addr + 32768u + (uint32_t)((nt * 4 + ks) * 1024));
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah[mt], bh.h, acc[mt][nt], 0, 0, 0);
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al[mt], bh.h, acc[mt][nt], 0, 0, 0);
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah[mt], bl.h, acc[mt][nt], 0, 0, 0);
        }
        // (the loops are unrolled because the accumulators are register arrays; without a fence
        // the scheduler hoists every B read of the step and spills)
        if (nt & 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- x norm, to float16, one 16-byte store per row: lane (col, g) holds elements 8 col + nt
    //      of rows 4g + i
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      const float nv[4] = {nr[mt].x, nr[mt].y, nr[mt].z, nr[mt].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        typedef typename akv_elem<ODT>::type out_t;
        out_t* orow;
        if constexpr (BLOCKS) {
          const int r = 16 * mt + 4 * g + i;
          if (row_p[r] < 0) continue;
          orow = (out_t*)a.out + row_o[r];
        } else {
          const int64_t r = base + 16 * mt + 4 * g + i;
          if (r >= a.n) continue;
          orow = (out_t*)a.out + r * a.os0;
        }
        // the reference multiplies the float32 rotated vector by the norm and then casts
        float v[8];
#pragma unroll
        for (int nt = 0; nt < 8; ++nt) v[nt] = __fmul_rn(acc[mt][nt][i] * (1.f / DM_PSCALE), nv[i]);
        if constexpr (ODT == AKV_F32) {
          *(float4*)(orow + 8 * col) = make_float4(v[0], v[1], v[2], v[3]);
          *(float4*)(orow + 8 * col + 4) = make_float4(v[4], v[5], v[6], v[7]);
        } else {
          uint32_t w[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if constexpr (ODT == AKV_F16) {
              w[q] = (uint32_t)__half_as_ushort(__float2half_rn(v[2 * q])) | ((uint32_t)__half_as_ushort(__float2half_rn(v[2 * q + 1])) << 16);
            } else {
              w[q] = (uint32_t)akv_float_to_bf16_bits(v[2 * q]) | ((uint32_t)akv_float_to_bf16_bits(v[2 * q + 1]) << 16);
            }
          }
          *(uint4*)(orow + 8 * col) = make_uint4(w[0], w[1], w[2], w[3]);
        }
      }
    }
  }
}

static bool dm_disabled() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("AKV_DISABLE_MFMA");
    v = (e && e[0] == '1') ? 1 : 0;
  }
  return v == 1;
}

// returns AKV_ERR_UNSUPPORTED when the fast path does not apply (the caller then uses the general kernel)
int akv_decode_mfma_try(const akv_gen_args& a, bool blocks, int d, int bits, int out_dtype, const void* rot_prep,
                        hipStream_t stream) {
  if (dm_disabled() || d != 128 || bits < 2 || bits > 4) return AKV_ERR_UNSUPPORTED;
  const uintptr_t palign = 3;      // a lane reads 16 / 12 / 8 bytes of a row: multi-dword loads need dword alignment only
  if ((((uintptr_t)a.packed | (uintptr_t)a.ps0) & palign) || ((uintptr_t)a.out & 15)) return AKV_ERR_UNSUPPORTED;
  if (a.os0 & 7) return AKV_ERR_UNSUPPORTED;      // rows of the output are written 8 elements (16 or 32 bytes) per lane
  if (blocks && (((uintptr_t)a.ps1 | (uintptr_t)a.ps2) & palign || ((a.os1 | a.os2) & 7))) return AKV_ERR_UNSUPPORTED;
  const uint4* bop = (const uint4*)((const char*)rot_prep + AKV_PREP_DECODE_OFFSET(d));
  const int64_t steps = (a.n + DM_ROWS - 1) / DM_ROWS;
  const int grid = (int)(steps < akv_cached_cu_count() ? steps : akv_cached_cu_count());
#define DM_GO(BL, BB, OD)                                                                                      \
  do {                                                                                                       \
    static bool configured = false;                                                                          \
    if (!configured) {                                                                                       \
      AKV_HIP(hipFuncSetAttribute((const void*)akv_decode_mfma_kernel<BL, BB, OD>,                           \
                                  hipFuncAttributeMaxDynamicSharedMemorySize, DM_LDS_BYTES));                \
      configured = true;                                                                                     \
    }                                                                                                        \
    AKV_LAUNCH_TIMED((akv_decode_mfma_kernel<BL, BB, OD>), grid, DM_THREADS, DM_LDS_BYTES, stream, a, bop);  \
  } while (0)
#define DM_GO_DT(BL, BB)                                                                                       \
  do {                                                                                                       \
    if (out_dtype == AKV_F16) DM_GO(BL, BB, AKV_F16);                                                        \
    else if (out_dtype == AKV_BF16) DM_GO(BL, BB, AKV_BF16);                                                 \
    else DM_GO(BL, BB, AKV_F32);                                                                             \
  } while (0)
  if (blocks) { if (bits == 4) DM_GO_DT(true, 4); else if (bits == 3) DM_GO_DT(true, 3); else DM_GO_DT(true, 2); }
  else { if (bits == 4) DM_GO_DT(false, 4); else if (bits == 3) DM_GO_DT(false, 3); else DM_GO_DT(false, 2); }
#undef DM_GO_DT
#undef DM_GO
  AKV_LAUNCH_CHECK("akv_decode_mfma_kernel");
  return AKV_OK;
}
