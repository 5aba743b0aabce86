// tq35 hybrid codec (head_dim 128, groups = dims 0..63 at 3-bit MSE and dims 64..127 at
// 2-bit MSE, each plus a 1-bit QJL residual sketch and two fp16 norms inside the 64-byte
// row): encode (flat / paged), decode, and decode attention directly on the packed rows.
//
// Row layout (aither_kvcache/hybrid_quantizer.py:92-123,771-779):
//   [0,24)  group-0 MSE codes, 3 bits each, MSB-first stream     [24,32) group-0 QJL sign bits
//   [32,34) group-0 norm fp16 LE    [34,36) group-0 residual norm fp16 LE
//   [36,52) group-1 MSE codes, 2 bits each                        [52,60) group-1 QJL sign bits
//   [60,62) group-1 norm            [62,64) group-1 residual norm
//
// With Fwd_s(z) = H(s.z)/8 and Inv_s(z) = s.H(z)/8 (H = 64-point Walsh-Hadamard, H H = 64 I)
// a decoded group is  n (Inv_had(c[idx]) + rho kappa Inv_qjl(sigma)),  kappa = sqrt(pi/2)/64.
// Because H is symmetric, <q, Inv_s(z)> = <Fwd_s(q), z>: attention scores are taken against
// the codes and sign bits directly with four transformed copies of the query, and the value
// sum is accumulated in the four transformed domains and inverted once at the end.
#include "akv_attn_common.h"
#include "akv_hybrid_layout.h"

static bool hyb_lane_disabled();
static bool hyb_lane_forced();
static const float kHybKappa = (float)(1.2533141373155001 / 64.0);  // sqrt(pi/2) / 64

__device__ __forceinline__ float hyb_half_bits_to_float(uint32_t b) {
  return __half2float(__ushort_as_half((unsigned short)(b & 0xffffu)));
}

// ----------------------------------------------------------------------------------
// encode: one wavefront per vector, lanes <-> coordinates of a group
// ----------------------------------------------------------------------------------
struct hyb_enc_args {
  const void* x; int64_t n; int64_t xs0, xs1; int heads;
  const void* x2; uint8_t* out2;     // paged, wavefront per vector: a second tensor (V beside K) with the same strides, or null
  const void* slots; int slot_itype; int block_size; int64_t max_blocks;
  const float* table;
  uint8_t* out; int64_t ps0, ps1, ps2;
};

template <int MB>
__device__ __forceinline__ void hyb_encode_group(float xv, int lane, const float* had, const float* qjl,
                                                 const float* cen, const float* bnd,
                                                 uint8_t* codes, uint8_t* signs, uint8_t* row,
                                                 int row_off) {
  const float ss = akv_wave_sum(akv_mul_rn(xv, xv));
  const float nrm = sqrtf(ss);
  const float unit = __fdiv_rn(xv, akv_add_rn(nrm, 1e-10f));
  const float rot = akv_mul_rn(hyb_fwht64(akv_mul_rn(unit, had[lane]), lane), 0.125f);
  const uint32_t code = akv_search<MB>(rot, bnd);
  const float mse_hat = akv_mul_rn(akv_mul_rn(hyb_fwht64(cen[code], lane), had[lane]), 0.125f);
  const float res = akv_sub_rn(unit, mse_hat);
  const float rn = sqrtf(akv_wave_sum(akv_mul_rn(res, res)));
  const float proj = akv_mul_rn(hyb_fwht64(akv_mul_rn(res, qjl[lane]), lane), 0.125f);
  codes[lane] = (uint8_t)code;
  signs[lane] = proj >= 0.f ? 1 : 0;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  constexpr int MSE_BYTES = 64 * MB / 8;
  if (lane < MSE_BYTES)
    row[row_off + lane] = (uint8_t)akv_stream_byte<MB>(lane, [&](int d) { return (uint32_t)codes[d]; });
  if (lane < 8)
    row[row_off + MSE_BYTES + lane] = (uint8_t)akv_stream_byte<1>(lane, [&](int d) { return (uint32_t)signs[d]; });
  if (lane == 0) {
    const unsigned short nb = __half_as_ushort(__float2half_rn(nrm));
    const unsigned short rb = __half_as_ushort(__float2half_rn(rn));
    row[row_off + MSE_BYTES + 8] = (uint8_t)(nb & 0xff);
    row[row_off + MSE_BYTES + 9] = (uint8_t)(nb >> 8);
    row[row_off + MSE_BYTES + 10] = (uint8_t)(rb & 0xff);
    row[row_off + MSE_BYTES + 11] = (uint8_t)(rb >> 8);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int XDT, bool PAGED>
__global__ __launch_bounds__(256) void hyb_encode_kernel(hyb_enc_args a) {
  __shared__ float tab[AKV_HYB_TABLE_FLOATS];
  __shared__ uint8_t codes[4][64], signs[4][64], rows[4][64];
  for (int i = threadIdx.x; i < AKV_HYB_TABLE_FLOATS; i += 256) tab[i] = a.table[i];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t n_total = (PAGED && a.x2) ? 2 * a.n : a.n;
  for (int64_t nn = (int64_t)blockIdx.x * 4 + wave; nn < n_total; nn += (int64_t)gridDim.x * 4) {
    const bool second = PAGED && nn >= a.n;                     // (wavefront-uniform)
    const int64_t n = second ? nn - a.n : nn;
    const void* xb = second ? a.x2 : a.x;
    const int64_t off = PAGED ? (n / a.heads) * a.xs0 + (n % a.heads) * a.xs1 : n * a.xs0;
    const float x0 = akv_elem<XDT>::load(xb, off + lane);
    const float x1 = akv_elem<XDT>::load(xb, off + 64 + lane);
    hyb_encode_group<3>(x0, lane, tab + HYB_HAD0, tab + HYB_QJL0, tab + HYB_CEN0, tab + HYB_BND0,
                        codes[wave], signs[wave], rows[wave], 0);
    hyb_encode_group<2>(x1, lane, tab + HYB_HAD1, tab + HYB_QJL1, tab + HYB_CEN1, tab + HYB_BND1,
                        codes[wave], signs[wave], rows[wave], 36);
    uint8_t* dst;
    if (PAGED) {
      const int64_t tok = n / a.heads, head = n % a.heads;
      const int64_t slot = akv_load_index(a.slots, a.slot_itype, tok);
      if (slot < 0) continue;
      const int64_t blk = slot / a.block_size, pos = slot % a.block_size;
      if (blk >= a.max_blocks) continue;
      dst = (second ? a.out2 : a.out) + blk * a.ps0 + pos * a.ps1 + head * a.ps2;
    } else {
      dst = a.out + n * a.ps0;
    }
    dst[lane] = rows[wave][lane];
  }
}

// ----------------------------------------------------------------------------------
// encode, one LANE per vector (rows of 16-byte aligned input and output): the 64-point transforms run
// in the lane's registers, so no lane ever talks to another -- 384 additions per transform where the
// wavefront-per-vector form above spends six shuffles per coordinate for one vector at a time.  Every
// operation, the order of the butterflies and the order of the sums are those of the kernel above
// (and of the reference); only the division is a reciprocal with one correction step.
// ----------------------------------------------------------------------------------
// (The reference rounds every operation: the products come from akv_mul_rn, which the compiler may not
// fuse into a multiply-add.  Where a product that is not exact feeds a tree of sums it also passes
// through hyb_rounded(), an empty asm statement the optimiser cannot see through, so the tree is not
// reassociated around it either.)
__device__ __forceinline__ float hyb_rounded(float x) {
  asm volatile("" : "+v"(x));
  return x;
}
__device__ __forceinline__ void hyb_fwht64_regs(float (&v)[64]) {
#pragma unroll
  for (int h = 1; h < 64; h <<= 1)
#pragma unroll
    for (int i = 0; i < 64; ++i)
      if ((i & h) == 0) {
        const float lo = v[i], hi = v[i + h];
        v[i] = akv_add_rn(lo, hi);
        v[i + h] = akv_sub_rn(lo, hi);
      }
}
// sum in the order of the wavefront reduction (partners 32, 16, ..., 1 apart)
__device__ __forceinline__ float hyb_tree_sum64(float (&t)[64]) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1)
#pragma unroll
    for (int i = 0; i < m; ++i) t[i] = akv_add_rn(t[i], t[i + m]);
  return t[0];
}
__device__ __forceinline__ void hyb_put_byte(uint32_t* words, int k, uint32_t byte) { words[k >> 2] |= byte << (8 * (k & 3)); }

// one group of 64 coordinates of the lane's vector -> MB-bit codes, sign bits and the two norms as
// dwords of the packed row (6 / 4 dwords of codes, 2 of signs, 1 of norms)
template <int XDT, int MB>
__device__ __forceinline__ void hyb_encode_group_lane(const void* x, int64_t off, const float* had,
                                                       const float* qjl, const float* cen, const float* bnd,
                                                       uint32_t* words) {
  constexpr int CW = 64 * MB / 32;       // dwords of codes
  float u[64], v[64];
  if constexpr (XDT == AKV_F32) {
    const float4* p = (const float4*)((const float*)x + off);
#pragma unroll
    for (int i = 0; i < 16; ++i) { const float4 q = p[i]; u[4 * i] = q.x; u[4 * i + 1] = q.y; u[4 * i + 2] = q.z; u[4 * i + 3] = q.w; }
  } else {
    const uint4* p = (const uint4*)((const unsigned short*)x + off);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint4 q = p[i];
      const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (XDT == AKV_F16) {
          u[8 * i + 2 * j] = __half2float(__ushort_as_half((unsigned short)(w[j] & 0xffffu)));
          u[8 * i + 2 * j + 1] = __half2float(__ushort_as_half((unsigned short)(w[j] >> 16)));
        } else {
          u[8 * i + 2 * j] = __uint_as_float(w[j] << 16);
          u[8 * i + 2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 64; ++j) v[j] = hyb_rounded(akv_mul_rn(u[j], u[j]));
  const float nrm = sqrtf(hyb_tree_sum64(v));
  const float den = akv_add_rn(nrm, 1e-10f);
  const float rcp = __frcp_rn(den);
  const bool plain = !(den < INFINITY);
#pragma unroll
  for (int j = 0; j < 64; ++j) {
    // x / den: reciprocal, then one correction step (the correctly rounded quotient but for rare ties)
    const float q0 = akv_mul_rn(u[j], rcp);
    const float e = fmaf(-q0, den, u[j]);
    // (an infinite or NaN norm: x * (1 / den) alone already is what the division gives)
    const float q = plain ? q0 : fmaf(e, rcp, q0);
    u[j] = q;
    v[j] = akv_mul_rn(q, had[j]);
  }
  hyb_fwht64_regs(v);
#pragma unroll
  for (int k = 0; k < CW + 3; ++k) words[k] = 0u;
  // codes: MSB-first stream; the centroid of every code goes straight into the next transform
  if constexpr (MB == 3) {
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      uint32_t g24 = 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t c = akv_search<3>(akv_mul_rn(v[8 * g + i], 0.125f), bnd);
        g24 |= c << (21 - 3 * i);
        v[8 * g + i] = cen[c];
      }
      hyb_put_byte(words, 3 * g, g24 >> 16);
      hyb_put_byte(words, 3 * g + 1, (g24 >> 8) & 0xffu);
      hyb_put_byte(words, 3 * g + 2, g24 & 0xffu);
    }
  } else {
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      uint32_t b = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t c = akv_search<2>(akv_mul_rn(v[4 * k + i], 0.125f), bnd);
        b |= c << (6 - 2 * i);
        v[4 * k + i] = cen[c];
      }
      hyb_put_byte(words, k, b);
    }
  }
  hyb_fwht64_regs(v);
#pragma unroll
  for (int j = 0; j < 64; ++j) {
    const float mse_hat = akv_mul_rn(akv_mul_rn(v[j], had[j]), 0.125f);
    u[j] = akv_sub_rn(u[j], mse_hat);              // residual
    v[j] = hyb_rounded(akv_mul_rn(u[j], u[j]));
  }
  const float rn = sqrtf(hyb_tree_sum64(v));
#pragma unroll
  for (int j = 0; j < 64; ++j) v[j] = akv_mul_rn(u[j], qjl[j]);
  hyb_fwht64_regs(v);
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    uint32_t b = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) b |= (akv_mul_rn(v[8 * k + i], 0.125f) >= 0.f ? 1u : 0u) << (7 - i);
    hyb_put_byte(words + CW, k, b);
  }
  words[CW + 2] = (uint32_t)__half_as_ushort(__float2half_rn(nrm)) | ((uint32_t)__half_as_ushort(__float2half_rn(rn)) << 16);
}

template <int XDT, bool PAGED>
__global__ __launch_bounds__(256) void hyb_encode_lane_kernel(hyb_enc_args a) {
  __shared__ float tab[AKV_HYB_TABLE_FLOATS];
  for (int i = threadIdx.x; i < AKV_HYB_TABLE_FLOATS; i += 256) tab[i] = a.table[i];
  __syncthreads();
  const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (n >= a.n) return;
  uint8_t* dst;
  int64_t off;
  if (PAGED) {
    const int64_t tok = n / a.heads, head = n - tok * a.heads;
    off = tok * a.xs0 + head * a.xs1;
    const int64_t slot = akv_load_index(a.slots, a.slot_itype, tok);
    if (slot < 0) return;
    const int64_t blk = slot / a.block_size, pos = slot - blk * a.block_size;
    if (blk >= a.max_blocks) return;
    dst = a.out + blk * a.ps0 + pos * a.ps1 + head * a.ps2;
  } else {
    off = n * a.xs0;
    dst = a.out + n * a.ps0;
  }
  uint32_t row[16];
  hyb_encode_group_lane<XDT, 3>(a.x, off, tab + HYB_HAD0, tab + HYB_QJL0, tab + HYB_CEN0, tab + HYB_BND0, row);
  hyb_encode_group_lane<XDT, 2>(a.x, off + 64, tab + HYB_HAD1, tab + HYB_QJL1, tab + HYB_CEN1, tab + HYB_BND1, row + 9);
  uint4* d4 = (uint4*)dst;
#pragma unroll
  for (int i = 0; i < 4; ++i) d4[i] = make_uint4(row[4 * i], row[4 * i + 1], row[4 * i + 2], row[4 * i + 3]);
}

// ----------------------------------------------------------------------------------
// decode: one wavefront per vector
// ----------------------------------------------------------------------------------
template <int MB>
__device__ __forceinline__ float hyb_decode_group(const uint8_t* row, int lane, const float* had,
                                                  const float* qjl, const float* cen, float kappa) {
  constexpr int MSE_BYTES = 64 * MB / 8;
  const uint32_t code = akv_stream_code<MB>(lane, [&](int o) { return (uint32_t)row[o]; });
  const float mse_hat = akv_mul_rn(akv_mul_rn(hyb_fwht64(cen[code], lane), had[lane]), 0.125f);
  const uint32_t bit = (row[MSE_BYTES + (lane >> 3)] >> (7 - (lane & 7))) & 1u;
  const float sg = bit ? kappa : -kappa;
  const float qjl_hat = akv_mul_rn(akv_mul_rn(hyb_fwht64(sg, lane), qjl[lane]), 0.125f);
  const float n = hyb_half_bits_to_float(row[MSE_BYTES + 8] | (row[MSE_BYTES + 9] << 8));
  const float rn = hyb_half_bits_to_float(row[MSE_BYTES + 10] | (row[MSE_BYTES + 11] << 8));
  return akv_mul_rn(akv_add_rn(mse_hat, akv_mul_rn(qjl_hat, rn)), n);
}

__global__ __launch_bounds__(256) void hyb_decode_kernel(const uint8_t* __restrict__ packed,
                                                         int64_t ps, int64_t n_vec,
                                                         const float* __restrict__ table, float kappa,
                                                         float* __restrict__ out, int64_t os) {
  __shared__ float tab[AKV_HYB_TABLE_FLOATS];
  __shared__ uint8_t rows[4][64];
  for (int i = threadIdx.x; i < AKV_HYB_TABLE_FLOATS; i += 256) tab[i] = table[i];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int64_t n = (int64_t)blockIdx.x * 4 + wave; n < n_vec; n += (int64_t)gridDim.x * 4) {
    rows[wave][lane] = packed[n * ps + lane];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    out[n * os + lane] = hyb_decode_group<3>(rows[wave], lane, tab + HYB_HAD0, tab + HYB_QJL0, tab + HYB_CEN0, kappa);
    out[n * os + 64 + lane] = hyb_decode_group<2>(rows[wave] + 36, lane, tab + HYB_HAD1, tab + HYB_QJL1, tab + HYB_CEN1, kappa);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// decode, one lane per vector (16-byte aligned rows): the same operations as above, transforms in registers
template <int MB>
__device__ __forceinline__ void hyb_decode_group_lane(const uint32_t* words, const float* had, const float* qjl,
                                                       const float* cen, float kappa, float* out) {
  constexpr int CW = 64 * MB / 32;
  auto byte_of = [&](int k) { return (words[k >> 2] >> (8 * (k & 3))) & 0xffu; };
  float v[64], w[64];
#pragma unroll
  for (int j = 0; j < 64; ++j) {
    v[j] = cen[akv_stream_code<MB>(j, byte_of)];
    const uint32_t bit = (byte_of(4 * CW + (j >> 3)) >> (7 - (j & 7))) & 1u;
    w[j] = bit ? kappa : -kappa;
  }
  hyb_fwht64_regs(v);
  hyb_fwht64_regs(w);
  const float n = hyb_half_bits_to_float(words[CW + 2]);
  const float rn = hyb_half_bits_to_float(words[CW + 2] >> 16);
#pragma unroll
  for (int j = 0; j < 64; ++j) {
    const float mse_hat = akv_mul_rn(akv_mul_rn(v[j], had[j]), 0.125f);
    const float qjl_hat = akv_mul_rn(akv_mul_rn(w[j], qjl[j]), 0.125f);
    v[j] = akv_mul_rn(akv_add_rn(mse_hat, hyb_rounded(akv_mul_rn(qjl_hat, rn))), n);
  }
  float4* o4 = (float4*)out;
#pragma unroll
  for (int i = 0; i < 16; ++i) o4[i] = make_float4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]);
}

__global__ __launch_bounds__(256) void hyb_decode_lane_kernel(const uint8_t* __restrict__ packed, int64_t ps,
                                                              int64_t n_vec, const float* __restrict__ table,
                                                              float kappa, float* __restrict__ out, int64_t os) {
  __shared__ float tab[AKV_HYB_TABLE_FLOATS];
  for (int i = threadIdx.x; i < AKV_HYB_TABLE_FLOATS; i += 256) tab[i] = table[i];
  __syncthreads();
  const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (n >= n_vec) return;
  uint32_t row[16];
  const uint4* p = (const uint4*)(packed + n * ps);
#pragma unroll
  for (int i = 0; i < 4; ++i) { const uint4 q = p[i]; row[4 * i] = q.x; row[4 * i + 1] = q.y; row[4 * i + 2] = q.z; row[4 * i + 3] = q.w; }
  hyb_decode_group_lane<3>(row, tab + HYB_HAD0, tab + HYB_QJL0, tab + HYB_CEN0, kappa, out + n * os);
  hyb_decode_group_lane<2>(row + 9, tab + HYB_HAD1, tab + HYB_QJL1, tab + HYB_CEN1, kappa, out + n * os + 64);
}

// ----------------------------------------------------------------------------------
// attention
// ----------------------------------------------------------------------------------
struct hyb_attn_args {
  const uint8_t* kc; int64_t kps_blk, kps_pos, kps_head;
  const uint8_t* vc; int64_t vps_blk, vps_pos, vps_head;
  const void* block_tables; int bt_itype; int64_t bt_stride;
  const void* context_lens; int cl_itype;
  const float* table;
  int S, QH, KVH, block_size;
  int64_t max_blocks_per_seq;
  int64_t num_blocks;  // physical blocks in the cache; table entries are clamped into [0, num_blocks)
  float scale, kappa;
  const int32_t* prefix;
  const float* qt;     // [S][QH][256]: Fwd_had(q0) | kappa Fwd_qjl(q0) | Fwd_had(q1) | kappa Fwd_qjl(q1)
  float* part_acc;     // [G+S][QH][256]: A0 | B0 | A1 | B1
  float* part_ml;
};

// prologue: 4 (sequence, query head) pairs per workgroup; the last workgroup does the prefix
template <int QDT>
__global__ __launch_bounds__(256) void hyb_attn_prologue_kernel(
    const void* __restrict__ query, int64_t qs_seq, int64_t qs_head, const float* __restrict__ table,
    float kappa, int S, int QH, const void* context_lens, int cl_itype, int block_size,
    int64_t max_blocks_per_seq, int32_t* prefix, float* __restrict__ qt, int nblocks_q,
    uint32_t* __restrict__ status) {
  __shared__ int32_t scratch[257];
  if ((int)blockIdx.x == nblocks_q) {
    if (threadIdx.x == 0) status[0] = 0u;
    akv_block_prefix_scan(context_lens, cl_itype, S, block_size, max_blocks_per_seq, prefix, scratch);
    return;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pair = blockIdx.x * 4 + wave;
  if (pair >= S * QH) return;
  const int s = pair / QH, h = pair % QH;
  const int64_t off = s * qs_seq + h * qs_head;
  const float q0 = akv_elem<QDT>::load(query, off + lane);
  const float q1 = akv_elem<QDT>::load(query, off + 64 + lane);
  float* o = qt + (size_t)pair * 256;
  o[lane] = hyb_fwht64(q0 * table[HYB_HAD0 + lane], lane) * 0.125f;
  o[64 + lane] = hyb_fwht64(q0 * table[HYB_QJL0 + lane], lane) * 0.125f * kappa;
  o[128 + lane] = hyb_fwht64(q1 * table[HYB_HAD1 + lane], lane) * 0.125f;
  o[192 + lane] = hyb_fwht64(q1 * table[HYB_QJL1 + lane], lane) * 0.125f * kappa;
}

#define HYB_WAVES 8
#define HYB_VROW 17

template <int GQ>
struct hyb_attn_cfg {
  static constexpr size_t wave_floats = 64 * GQ * 4 + 64 * HYB_VROW;
  static size_t lds_bytes(int QH) { return ((size_t)QH * 256 + HYB_WAVES * wave_floats + 16) * 4; }
};

template <int GQ>
__global__ __launch_bounds__(512) void hyb_attn_kernel(hyb_attn_args a) {
  typedef hyb_attn_cfg<GQ> cfg;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  float* q_lds = (float*)lds_raw;                          // [QH][256]
  float* wave_base = q_lds + (size_t)a.QH * 256;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* p_lds = wave_base + wave * cfg::wave_floats;      // [64][GQ][4]
  uint32_t* v_lds = (uint32_t*)(p_lds + 64 * GQ * 4);      // [64][17]
  float* cen = wave_base + HYB_WAVES * cfg::wave_floats;   // 8 + 4 centroids
  if (threadIdx.x < 12) cen[threadIdx.x] = a.table[HYB_CEN0 + threadIdx.x];
  const float* cen0 = cen;
  const float* cen1 = cen + 8;

  const int G = gridDim.x;
  const int total = a.prefix[a.S];
  const int per = (total + G - 1) / G;
  const int g0 = blockIdx.x * per;
  const int g1 = min(total, g0 + per);
  const int gqa = a.QH / a.KVH;
  const int bs = a.block_size;

  int g = g0;
  while (g < g1) {
    const int s = akv_find_seq(a.prefix, a.S, g);
    const int sb0 = a.prefix[s], sb1 = a.prefix[s + 1];
    const int blk_lo = g - sb0;
    const int blk_hi = min(g1, sb1) - sb0;
    const int64_t ctx = akv_seq_tokens(a.context_lens, a.cl_itype, s, bs, a.max_blocks_per_seq);
    const int t0 = blk_lo * bs;
    const int t1 = (int)min((int64_t)blk_hi * bs, ctx);
    g = sb0 + blk_hi;

    __syncthreads();
    for (int i = threadIdx.x; i < a.QH * 256; i += blockDim.x)
      q_lds[i] = a.qt[(size_t)s * a.QH * 256 + i];
    __syncthreads();

    for (int h = wave; h < a.KVH; h += HYB_WAVES) {
      for (int qg = 0; qg < gqa; qg += GQ) {
        float m[GQ], l[GQ], acc[GQ][4];
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          m[q] = -INFINITY; l[q] = 0.f;
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[q][i] = 0.f;
        }
        const float* qh = q_lds + (size_t)(h * gqa + qg) * 256;

        for (int c0 = t0; c0 < t1; c0 += 64) {
          const int t = c0 + lane;
          const bool valid = t < t1;
          const int tc = valid ? t : t1 - 1;
          const int64_t phys = akv_clamp_block(akv_load_index(a.block_tables, a.bt_itype, s * a.bt_stride + tc / bs), a.num_blocks);
          const int pos = tc % bs;
          uint32_t row[16];
          {
            const uint32_t* kr = (const uint32_t*)(a.kc + phys * a.kps_blk + pos * a.kps_pos + h * a.kps_head);
#pragma unroll
            for (int i = 0; i < 16; ++i) row[i] = kr[i];
          }
          auto kb = [&](int o) { return (row[o >> 2] >> (8 * (o & 3))) & 0xffu; };
          float d0[GQ], e0[GQ], d1[GQ], e1[GQ];
#pragma unroll
          for (int q = 0; q < GQ; ++q) { d0[q] = e0[q] = d1[q] = e1[q] = 0.f; }
#pragma unroll
          for (int j = 0; j < 64; ++j) {
            const float c0v = cen0[akv_stream_code<3>(j, kb)];
            const float s0v = ((kb(24 + (j >> 3)) >> (7 - (j & 7))) & 1u) ? 1.f : -1.f;
            const float c1v = cen1[akv_stream_code<2>(j, [&](int o) { return kb(36 + o); })];
            const float s1v = ((kb(52 + (j >> 3)) >> (7 - (j & 7))) & 1u) ? 1.f : -1.f;
#pragma unroll
            for (int q = 0; q < GQ; ++q) {
              d0[q] = fmaf(qh[q * 256 + j], c0v, d0[q]);
              e0[q] = fmaf(qh[q * 256 + 64 + j], s0v, e0[q]);
              d1[q] = fmaf(qh[q * 256 + 128 + j], c1v, d1[q]);
              e1[q] = fmaf(qh[q * 256 + 192 + j], s1v, e1[q]);
            }
          }
          const float kn0 = hyb_half_bits_to_float(row[8]), kr0 = hyb_half_bits_to_float(row[8] >> 16);
          const float kn1 = hyb_half_bits_to_float(row[15]), kr1 = hyb_half_bits_to_float(row[15] >> 16);
          // V row: registers -> norms, LDS -> codes
          uint32_t vrow[16];
          {
            const uint32_t* vr = (const uint32_t*)(a.vc + phys * a.vps_blk + pos * a.vps_pos + h * a.vps_head);
#pragma unroll
            for (int i = 0; i < 16; ++i) { vrow[i] = vr[i]; v_lds[lane * HYB_VROW + i] = vrow[i]; }
          }
          const float vn0 = hyb_half_bits_to_float(vrow[8]), vr0 = hyb_half_bits_to_float(vrow[8] >> 16);
          const float vn1 = hyb_half_bits_to_float(vrow[15]), vr1 = hyb_half_bits_to_float(vrow[15] >> 16);
#pragma unroll
          for (int q = 0; q < GQ; ++q) {
            const float raw = kn0 * (d0[q] + kr0 * e0[q]) + kn1 * (d1[q] + kr1 * e1[q]);
            const float sv = valid ? raw * a.scale : -INFINITY;
            const float mt = akv_wave_max(sv);
            const float mn = fmaxf(m[q], mt);
            const float alpha = __expf(m[q] - mn);
            const float p = valid ? __expf(sv - mn) : 0.f;
            l[q] = l[q] * alpha + p;
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[q][i] *= alpha;
            m[q] = mn;
            float4 pw;
            pw.x = p * vn0; pw.y = p * vn0 * vr0 * a.kappa; pw.z = p * vn1; pw.w = p * vn1 * vr1 * a.kappa;
            *(float4*)(p_lds + (lane * GQ + q) * 4) = pw;
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          const int nt = min(64, t1 - c0);
          for (int tt = 0; tt < nt; ++tt) {
            const uint8_t* vb = (const uint8_t*)(v_lds + tt * HYB_VROW);
            const float c0v = cen0[akv_stream_code<3>(lane, [&](int o) { return (uint32_t)vb[o]; })];
            const float s0v = ((vb[24 + (lane >> 3)] >> (7 - (lane & 7))) & 1u) ? 1.f : -1.f;
            const float c1v = cen1[akv_stream_code<2>(lane, [&](int o) { return (uint32_t)vb[36 + o]; })];
            const float s1v = ((vb[52 + (lane >> 3)] >> (7 - (lane & 7))) & 1u) ? 1.f : -1.f;
#pragma unroll
            for (int q = 0; q < GQ; ++q) {
              const float4 pw = *(const float4*)(p_lds + (tt * GQ + q) * 4);
              acc[q][0] = fmaf(pw.x, c0v, acc[q][0]);
              acc[q][1] = fmaf(pw.y, s0v, acc[q][1]);
              acc[q][2] = fmaf(pw.z, c1v, acc[q][2]);
              acc[q][3] = fmaf(pw.w, s1v, acc[q][3]);
            }
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          const size_t slot = (size_t)(blockIdx.x + s) * a.QH + (h * gqa + qg + q);
          const float lsum = akv_wave_sum(l[q]);
#pragma unroll
          for (int i = 0; i < 4; ++i) a.part_acc[slot * 256 + i * 64 + lane] = acc[q][i];
          if (lane == 0) { a.part_ml[slot * 2] = m[q]; a.part_ml[slot * 2 + 1] = lsum; }
        }
      }
    }
  }
}

template <int ODT>
__global__ __launch_bounds__(64) void hyb_attn_reduce_kernel(
    const int32_t* __restrict__ prefix, const float* __restrict__ part_acc,
    const float* __restrict__ part_ml, const float* __restrict__ table, int S, int QH, int G,
    void* __restrict__ out, int64_t os_seq, int64_t os_head, const uint32_t* __restrict__ status) {
  const int s = blockIdx.x / QH, h = blockIdx.x % QH;
  const int lane = threadIdx.x;
  const int b0 = prefix[s], b1 = prefix[s + 1];
  const int64_t obase = s * os_seq + h * os_head;
  // a main kernel whose bounded wait gave up has produced garbage: say so in every output
  const float poison = status[0] != 0u ? __uint_as_float(0x7fc00000u) : 0.f;
  if (b1 <= b0) {
    akv_elem<ODT>::store(out, obase + lane, poison);
    akv_elem<ODT>::store(out, obase + 64 + lane, poison);
    return;
  }
  const int total = prefix[S];
  const int per = (total + G - 1) / G;
  const int w_lo = b0 / per, w_hi = (b1 - 1) / per;
  float m = -INFINITY, l = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int w = w_lo; w <= w_hi; ++w) {
    const size_t slot = (size_t)(w + s) * QH + h;
    float alpha, beta;
    akv_lse_merge(m, l, part_ml[slot * 2], part_ml[slot * 2 + 1], alpha, beta);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = alpha * acc[i] + beta * part_acc[slot * 256 + i * 64 + lane];
  }
  const float inv = l > 0.f ? 1.f / l : 1.f;
  const float o0 = (hyb_fwht64(acc[0] * inv, lane) * table[HYB_HAD0 + lane] +
                    hyb_fwht64(acc[1] * inv, lane) * table[HYB_QJL0 + lane]) * 0.125f;
  const float o1 = (hyb_fwht64(acc[2] * inv, lane) * table[HYB_HAD1 + lane] +
                    hyb_fwht64(acc[3] * inv, lane) * table[HYB_QJL1 + lane]) * 0.125f;
  akv_elem<ODT>::store(out, obase + lane, o0 + poison);
  akv_elem<ODT>::store(out, obase + 64 + lane, o1 + poison);
}

// ----------------------------------------------------------------------------------
// host entries
// ----------------------------------------------------------------------------------
static int hyb_grid(int64_t n) {
  int cus = akv_cached_cu_count();
  int64_t cap = (int64_t)(cus > 0 ? cus : 256) * 8;
  int64_t g = (n + 3) / 4;
  return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

static bool hyb_lane_forced() {
  const char* e = getenv("AKV_HYBRID_LANE_ENCODE");        // (read per call: tests switch it)
  return e && e[0] == '1';
}

static bool hyb_lane_disabled() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("AKV_HYBRID_WAVE_ENCODE");
    v = (e && e[0] == '1') ? 1 : 0;
  }
  return v == 1;
}

template <bool PAGED>
static int hyb_launch_encode(int dt, const hyb_enc_args& a, hipStream_t stream) {
  // 16-byte aligned input rows and packed rows: one lane per vector
  const int64_t xal = dt == AKV_F32 ? 3 : 7;      // elements per 16 bytes, minus one
  // ... and enough of them: a lane walks its vector's six transforms alone (20 us however few vectors there are),
  // a wavefront per vector takes 7 us for a serving step of 2,048 vectors and 0.8 ns more per vector; they meet
  // near 16 K vectors
  const bool lane_form = (((uintptr_t)a.x | (uintptr_t)a.out | (uintptr_t)a.ps0 | (uintptr_t)(PAGED ? a.ps1 | a.ps2 : 0)) & 15) == 0 &&
                         ((a.xs0 | (PAGED ? a.xs1 : 0)) & xal) == 0 && !hyb_lane_disabled() &&
                         (a.n >= 16384 || hyb_lane_forced()) && a.x2 == nullptr;
  if (lane_form) {
    const int lgrid = (int)((a.n + 255) / 256);
    switch (dt) {
      case AKV_F16: hyb_encode_lane_kernel<AKV_F16, PAGED><<<lgrid, 256, 0, stream>>>(a); break;
      case AKV_BF16: hyb_encode_lane_kernel<AKV_BF16, PAGED><<<lgrid, 256, 0, stream>>>(a); break;
      default: hyb_encode_lane_kernel<AKV_F32, PAGED><<<lgrid, 256, 0, stream>>>(a); break;
    }
    AKV_LAUNCH_CHECK("hyb_encode_lane_kernel");
    return AKV_OK;
  }
  const int grid = hyb_grid((PAGED && a.x2) ? 2 * a.n : a.n);
  switch (dt) {
    case AKV_F16: hyb_encode_kernel<AKV_F16, PAGED><<<grid, 256, 0, stream>>>(a); break;
    case AKV_BF16: hyb_encode_kernel<AKV_BF16, PAGED><<<grid, 256, 0, stream>>>(a); break;
    default: hyb_encode_kernel<AKV_F32, PAGED><<<grid, 256, 0, stream>>>(a); break;
  }
  AKV_LAUNCH_CHECK("hyb_encode_kernel");
  return AKV_OK;
}

extern "C" int akv_hybrid_encode(const void* x, int x_dtype, int64_t n, int64_t x_stride,
                                 const float* hyb_table, uint8_t* out, int64_t out_stride_bytes,
                                 void* stream) {
  AKV_REQUIRE(n >= 0 && akv_valid_dtype(x_dtype), "akv_hybrid_encode: bad n / dtype");
  if (n == 0) return AKV_OK;
  AKV_REQUIRE(x && hyb_table && out, "akv_hybrid_encode: null pointer");
  AKV_REQUIRE(x_stride >= 128 && out_stride_bytes >= 64, "akv_hybrid_encode: stride smaller than row");
  hyb_enc_args a = {};
  a.x = x; a.n = n; a.xs0 = x_stride; a.heads = 1; a.table = hyb_table;
  a.out = out; a.ps0 = out_stride_bytes;
  return hyb_launch_encode<false>(x_dtype, a, (hipStream_t)stream);
}

extern "C" int akv_hybrid_encode_paged(const void* x, int x_dtype, int64_t num_tokens,
                                       int num_kv_heads, int64_t xs_token, int64_t xs_head,
                                       const void* slot_mapping, int slot_itype,
                                       const float* hyb_table, uint8_t* out, int64_t ps_blk,
                                       int64_t ps_pos, int64_t ps_head, int block_size,
                                       int64_t max_blocks, void* stream) {
  AKV_REQUIRE(num_tokens >= 0 && num_kv_heads > 0, "akv_hybrid_encode_paged: bad sizes");
  AKV_REQUIRE(akv_valid_dtype(x_dtype) && akv_valid_itype(slot_itype), "akv_hybrid_encode_paged: bad dtype");
  AKV_REQUIRE(block_size > 0 && max_blocks >= 0, "akv_hybrid_encode_paged: bad block_size/max_blocks");
  if (num_tokens == 0 || max_blocks == 0) return AKV_OK;
  AKV_REQUIRE(x && slot_mapping && hyb_table && out, "akv_hybrid_encode_paged: null pointer");
  hyb_enc_args a = {};
  a.x = x; a.n = num_tokens * num_kv_heads; a.xs0 = xs_token; a.xs1 = xs_head; a.heads = num_kv_heads;
  a.slots = slot_mapping; a.slot_itype = slot_itype; a.block_size = block_size; a.max_blocks = max_blocks;
  a.table = hyb_table; a.out = out; a.ps0 = ps_blk; a.ps1 = ps_pos; a.ps2 = ps_head;
  return hyb_launch_encode<true>(x_dtype, a, (hipStream_t)stream);
}

// K and V of a step in one launch while the call is small (a wavefront per vector); two launches of the form
// for large calls otherwise.  Both tensors and both caches have the strides given.
extern "C" int akv_hybrid_encode_paged_kv(const void* x_k, const void* x_v, int x_dtype, int64_t num_tokens,
                                          int num_kv_heads, int64_t xs_token, int64_t xs_head,
                                          const void* slot_mapping, int slot_itype,
                                          const float* hyb_table, uint8_t* out_k, uint8_t* out_v, int64_t ps_blk,
                                          int64_t ps_pos, int64_t ps_head, int block_size,
                                          int64_t max_blocks, void* stream) {
  AKV_REQUIRE(num_tokens >= 0 && num_kv_heads > 0, "akv_hybrid_encode_paged_kv: bad sizes");
  if (num_tokens == 0 || max_blocks == 0) return AKV_OK;
  AKV_REQUIRE(x_k && x_v && out_k && out_v, "akv_hybrid_encode_paged_kv: null pointer");
  if (num_tokens * num_kv_heads >= 16384) {
    const int rc = akv_hybrid_encode_paged(x_k, x_dtype, num_tokens, num_kv_heads, xs_token, xs_head, slot_mapping,
                                           slot_itype, hyb_table, out_k, ps_blk, ps_pos, ps_head, block_size, max_blocks, stream);
    if (rc) return rc;
    return akv_hybrid_encode_paged(x_v, x_dtype, num_tokens, num_kv_heads, xs_token, xs_head, slot_mapping,
                                   slot_itype, hyb_table, out_v, ps_blk, ps_pos, ps_head, block_size, max_blocks, stream);
  }
  AKV_REQUIRE(akv_valid_dtype(x_dtype) && akv_valid_itype(slot_itype), "akv_hybrid_encode_paged_kv: bad dtype");
  AKV_REQUIRE(block_size > 0 && max_blocks >= 0, "akv_hybrid_encode_paged_kv: bad block_size/max_blocks");
  AKV_REQUIRE(slot_mapping && hyb_table, "akv_hybrid_encode_paged_kv: null pointer");
  hyb_enc_args a = {};
  a.x = x_k; a.x2 = x_v; a.n = num_tokens * num_kv_heads; a.xs0 = xs_token; a.xs1 = xs_head; a.heads = num_kv_heads;
  a.slots = slot_mapping; a.slot_itype = slot_itype; a.block_size = block_size; a.max_blocks = max_blocks;
  a.table = hyb_table; a.out = out_k; a.out2 = out_v; a.ps0 = ps_blk; a.ps1 = ps_pos; a.ps2 = ps_head;
  return hyb_launch_encode<true>(x_dtype, a, (hipStream_t)stream);
}

extern "C" int akv_hybrid_decode(const uint8_t* packed, int64_t packed_stride_bytes, int64_t n,
                                 const float* hyb_table, float* out, int64_t out_stride,
                                 void* stream) {
  AKV_REQUIRE(n >= 0, "akv_hybrid_decode: n=%lld", (long long)n);
  if (n == 0) return AKV_OK;
  AKV_REQUIRE(packed && hyb_table && out, "akv_hybrid_decode: null pointer");
  AKV_REQUIRE(packed_stride_bytes >= 64 && out_stride >= 128, "akv_hybrid_decode: stride smaller than row");
  // (a lane per vector from 64 K vectors on; below that a wavefront per vector ends two to three microseconds earlier)
  if (!hyb_lane_disabled() && (((uintptr_t)packed | (uintptr_t)packed_stride_bytes | (uintptr_t)out) & 15) == 0 &&
      (out_stride & 3) == 0 && (n >= 65536 || hyb_lane_forced())) {
    hyb_decode_lane_kernel<<<(int)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(packed, packed_stride_bytes, n,
                                                                                  hyb_table, kHybKappa, out, out_stride);
    AKV_LAUNCH_CHECK("hyb_decode_lane_kernel");
    return AKV_OK;
  }
  hyb_decode_kernel<<<hyb_grid(n), 256, 0, (hipStream_t)stream>>>(packed, packed_stride_bytes, n, hyb_table,
                                                                  kHybKappa, out, out_stride);
  AKV_LAUNCH_CHECK("hyb_decode_kernel");
  return AKV_OK;
}

extern "C" size_t akv_hybrid_paged_attn_workspace_bytes(int num_seqs, int num_q_heads) {
  if (num_seqs < 0 || num_q_heads <= 0) return 0;
  return akv_attn_ws_layout(nullptr, num_seqs, num_q_heads, 256, akv_attn_grid()).bytes +
         akv_hyb_mfma_extra_bytes(num_seqs, num_q_heads);
}

template <int GQ>
static int hyb_launch_attn(const hyb_attn_args& a, int grid, hipStream_t stream) {
  const size_t lds = hyb_attn_cfg<GQ>::lds_bytes(a.QH);
  if (lds > 160 * 1024)
    return akv_fail(AKV_ERR_UNSUPPORTED, "hybrid_paged_attn: too many query heads for LDS (%zu bytes)", lds);
  AKV_HIP(hipFuncSetAttribute((const void*)hyb_attn_kernel<GQ>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  akv_profile_mark_begin(stream);
  hyb_attn_kernel<GQ><<<grid, 512, lds, stream>>>(a);
  akv_profile_mark_end(stream);
  AKV_LAUNCH_CHECK("hyb_attn_kernel");
  return AKV_OK;
}

extern "C" int akv_hybrid_paged_attn(
    const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head,
    const uint8_t* k_cache, int64_t kps_blk, int64_t kps_pos, int64_t kps_head,
    const uint8_t* v_cache, int64_t vps_blk, int64_t vps_pos, int64_t vps_head,
    const void* block_tables, int bt_itype, int64_t bt_stride,
    const void* context_lens, int cl_itype, const float* hyb_table,
    void* out, int out_dtype, int64_t os_seq, int64_t os_head,
    int num_seqs, int num_q_heads, int num_kv_heads,
    int block_size, int64_t num_blocks, int64_t max_blocks_per_seq, float scale,
    void* workspace, size_t workspace_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  AKV_REQUIRE(num_seqs >= 0 && num_q_heads > 0 && num_kv_heads > 0, "akv_hybrid_paged_attn: bad head/seq counts");
  AKV_REQUIRE((num_blocks > 0 && num_blocks < ((int64_t)1 << 31)) || max_blocks_per_seq == 0,
              "akv_hybrid_paged_attn: num_blocks=%lld with a non-empty block table", (long long)num_blocks);
  AKV_REQUIRE(num_q_heads % num_kv_heads == 0, "akv_hybrid_paged_attn: num_q_heads %% num_kv_heads != 0");
  AKV_REQUIRE(akv_valid_dtype(q_dtype) && akv_valid_dtype(out_dtype), "akv_hybrid_paged_attn: bad dtype");
  AKV_REQUIRE(akv_valid_itype(bt_itype) && akv_valid_itype(cl_itype), "akv_hybrid_paged_attn: bad index type");
  AKV_REQUIRE(block_size > 0 && max_blocks_per_seq >= 0, "akv_hybrid_paged_attn: bad block_size / table width");
  if (num_seqs == 0) return AKV_OK;
  AKV_REQUIRE(query && out && hyb_table && context_lens, "akv_hybrid_paged_attn: null pointer");
  AKV_REQUIRE(max_blocks_per_seq == 0 || (k_cache && v_cache && block_tables), "akv_hybrid_paged_attn: null cache pointer");
  AKV_REQUIRE((((uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)kps_blk | (uintptr_t)kps_pos |
                (uintptr_t)kps_head | (uintptr_t)vps_blk | (uintptr_t)vps_pos | (uintptr_t)vps_head) & 3) == 0,
              "akv_hybrid_paged_attn: packed rows must be 4-byte aligned");
  const int G = akv_attn_grid();
  AKV_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0, "akv_hybrid_paged_attn: workspace null or not 256-byte aligned");
  akv_attn_ws ws = akv_attn_ws_layout(workspace, num_seqs, num_q_heads, 256, G);
  const size_t need = ws.bytes + akv_hyb_mfma_extra_bytes(num_seqs, num_q_heads);
  if (workspace_bytes < need)
    return akv_fail(AKV_ERR_WORKSPACE, "akv_hybrid_paged_attn: workspace %zu < %zu bytes", workspace_bytes, need);

  // groups of four query heads over blocks of 16 or 32 tokens: the matrix-core kernel
  const int64_t strides6[6] = {kps_blk, kps_pos, kps_head, vps_blk, vps_pos, vps_head};
  const int rgrid = num_seqs * num_q_heads;
  int Gused = G;
  if (max_blocks_per_seq > 0 && akv_hyb_mfma_applicable(num_q_heads, num_kv_heads, block_size, strides6)) {
    akv_hyb_mfma_args m;
    m.kc = k_cache; m.kps_blk = kps_blk; m.kps_pos = kps_pos; m.kps_head = kps_head;
    m.vc = v_cache; m.vps_blk = vps_blk; m.vps_pos = vps_pos; m.vps_head = vps_head;
    m.block_tables = block_tables; m.bt_itype = bt_itype; m.bt_stride = bt_stride;
    m.context_lens = context_lens; m.cl_itype = cl_itype;
    m.S = num_seqs; m.QH = num_q_heads; m.KVH = num_kv_heads; m.hgroup = 1; m.block_size = block_size;
    m.max_blocks_per_seq = max_blocks_per_seq; m.num_blocks = num_blocks;
    m.prefix = ws.prefix; m.lut = nullptr; m.qop = nullptr; m.status = ws.status; m.spin_limit = 0;
    m.part_acc = ws.part_acc; m.part_ml = ws.part_ml;
    Gused = G / AKV_ATTN_WG_PER_CU;      // one workgroup per CU (its tables fill most of the LDS)
    const int rc = akv_hyb_mfma_run(query, q_dtype, qs_seq, qs_head, hyb_table, kHybKappa, scale, m, block_size,
                                    ws.prefix, ws.lut, (char*)workspace + ws.bytes, Gused, stream);
    if (rc) return rc;
  } else {

  const int nblocks_q = (num_seqs * num_q_heads + 3) / 4;
#define HYB_PRO(DT) hyb_attn_prologue_kernel<DT><<<nblocks_q + 1, 256, 0, stream>>>(query, qs_seq, qs_head, hyb_table, kHybKappa, num_seqs, num_q_heads, context_lens, cl_itype, block_size, max_blocks_per_seq, ws.prefix, ws.qrot, nblocks_q, ws.status)
  if (q_dtype == AKV_F16) HYB_PRO(AKV_F16); else if (q_dtype == AKV_BF16) HYB_PRO(AKV_BF16); else HYB_PRO(AKV_F32);
#undef HYB_PRO
  AKV_LAUNCH_CHECK("hyb_attn_prologue_kernel");

  hyb_attn_args a;
  a.kc = k_cache; a.kps_blk = kps_blk; a.kps_pos = kps_pos; a.kps_head = kps_head;
  a.vc = v_cache; a.vps_blk = vps_blk; a.vps_pos = vps_pos; a.vps_head = vps_head;
  a.block_tables = block_tables; a.bt_itype = bt_itype; a.bt_stride = bt_stride;
  a.context_lens = context_lens; a.cl_itype = cl_itype; a.table = hyb_table;
  a.S = num_seqs; a.QH = num_q_heads; a.KVH = num_kv_heads; a.block_size = block_size;
  a.max_blocks_per_seq = max_blocks_per_seq; a.num_blocks = num_blocks; a.scale = scale; a.kappa = kHybKappa;
  a.prefix = ws.prefix; a.qt = ws.qrot; a.part_acc = ws.part_acc; a.part_ml = ws.part_ml;
  const int gqa = num_q_heads / num_kv_heads;
  int rc = (gqa % 4 == 0) ? hyb_launch_attn<4>(a, G, stream) : hyb_launch_attn<1>(a, G, stream);
  if (rc) return rc;
  }
  switch (out_dtype) {
    case AKV_F16: hyb_attn_reduce_kernel<AKV_F16><<<rgrid, 64, 0, stream>>>(ws.prefix, ws.part_acc, ws.part_ml, hyb_table, num_seqs, num_q_heads, Gused, out, os_seq, os_head, ws.status); break;
    case AKV_BF16: hyb_attn_reduce_kernel<AKV_BF16><<<rgrid, 64, 0, stream>>>(ws.prefix, ws.part_acc, ws.part_ml, hyb_table, num_seqs, num_q_heads, Gused, out, os_seq, os_head, ws.status); break;
    default: hyb_attn_reduce_kernel<AKV_F32><<<rgrid, 64, 0, stream>>>(ws.prefix, ws.part_acc, ws.part_ml, hyb_table, num_seqs, num_q_heads, Gused, out, os_seq, os_head, ws.status); break;
  }
  AKV_LAUNCH_CHECK("hyb_attn_reduce_kernel");
  return AKV_OK;
}
