// tq25 hybrid codec (head_dim 128, calibrate_uniform groups: dims 0..31 at 2-bit MSE, dims 32..127 at
// 1-bit MSE, each plus a 1-bit QJL residual sketch and two fp16 norms inside the 44-byte row): encode
// (flat / paged), decode, and decode attention directly on the packed rows.
// aither_kvcache/hybrid_quantizer.py:59-65 (mode), :92-123 (layout), :616-779 (encode), :785-933 (decode).
//
// Row layout:
//   [0,8)   group-0 MSE codes, 2 bits each, MSB-first stream     [8,12)  group-0 QJL sign bits (bit 7 first)
//   [12,14) group-0 norm fp16 LE    [14,16) group-0 residual norm fp16 LE
//   [16,28) group-1 MSE codes, 1 bit each                         [28,40) group-1 QJL sign bits
//   [40,42) group-1 norm            [42,44) group-1 residual norm
//
// The 96 coordinates of group 1 are no power of two: the reference transforms them as a 64-point and a
// 32-point block, each unnormalised, and divides the whole group by sqrt(96) (fwht_general,
// hybrid_quantizer.py:154-193) -- the transform is not unitary there and is not made so here.  With
// Fwd_s(z) = H(s.z)/sqrt(dim) and Inv_s(z) = s.H(z)/sqrt(dim), H block diagonal and symmetric,
// <q, Inv_s(z)> = <Fwd_s(q), z> holds as for tq35: scores are taken against codes and sign bits with
// transformed copies of the query, the value sum is accumulated in the transformed domains and inverted
// once at the end.
//
// One wavefront per vector, two coordinates per lane: lane l holds coordinate 32 + l (the 64-point block of
// group 1) and, as its second value, coordinate l of group 0 (l < 32) or coordinate 64 + l of group 1's
// 32-point block (l >= 32) -- the two 32-point transforms are one butterfly over the lanes of each half.
#include "akv_attn_common.h"
#include "akv_hybrid_layout.h"

#define H25_HAD 0          // [128] Hadamard signs in coordinate order (group 0's 32, then group 1's 96)
#define H25_QJL 128        // [128] QJL signs likewise
#define H25_CEN0 256       // 4 centroids
#define H25_CEN1 260       // 2 centroids
#define H25_BND0 262       // 3 boundaries
#define H25_BND1 265       // 1 boundary
#define H25_ROW 44

// float32 values of sqrt(32), sqrt(96) and of sqrt(pi/2) / dim (hybrid_quantizer.py:232,540-541)
constexpr float kH25Root0 = 5.656854249492381f;
constexpr float kH25Root1 = 9.797958971132712f;
constexpr float kH25Kappa0 = (float)(1.2533141373155001 / 32.0);
constexpr float kH25Kappa1 = (float)(1.2533141373155001 / 96.0);

__device__ __forceinline__ float h25_half_bits_to_float(uint32_t b) {
  return __half2float(__ushort_as_half((unsigned short)(b & 0xffffu)));
}
// 32-point Walsh-Hadamard transform inside each half of the wavefront
__device__ __forceinline__ float h25_fwht32(float v, int lane) {
  v = hyb_fwht_step<1>(v, lane);
  v = hyb_fwht_step<2>(v, lane);
  v = hyb_fwht_step<4>(v, lane);
  v = hyb_fwht_step<8>(v, lane);
  v = hyb_fwht_step<16>(v, lane);
  return v;
}
// sum over the lanes of each half; every lane of a half receives its half's sum
__device__ __forceinline__ float h25_half_sum(float v) {
  v += akv_lane_xor<16>(v);
  v += akv_lane_xor<8>(v);
  v += akv_lane_xor<4>(v);
  v += akv_lane_xor<2>(v);
  v += akv_lane_xor<1>(v);
  return v;
}
__device__ __forceinline__ float h25_lane_value(float v, int src) {
  return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), src));
}

// the lane's two coordinates
struct h25_roles {
  int ca, cb;       // coordinate of the first value (group 1, 64-point block) and of the second
  bool b0;          // the second value belongs to group 0
  int ja, jb;       // position inside the group's code / sign streams
  __device__ __forceinline__ explicit h25_roles(int lane)
      : ca(32 + lane), cb(lane < 32 ? lane : 64 + lane), b0(lane < 32), ja(lane), jb(lane < 32 ? lane : 32 + lane) {}
};

// ----------------------------------------------------------------------------------
// encode
// ----------------------------------------------------------------------------------
struct h25_enc_args {
  const void* x; int64_t n; int64_t xs0, xs1; int heads;
  const void* x2; uint8_t* out2;     // paged: a second tensor (V beside K) with the same strides, or null
  const void* slots; int slot_itype; int block_size; int64_t max_blocks;
  const float* table;
  uint8_t* out; int64_t ps0, ps1, ps2;
};

template <int XDT, bool PAGED>
__global__ __launch_bounds__(256) void h25_encode_kernel(h25_enc_args a) {
  __shared__ float tab[AKV_HYB_TABLE_FLOATS];
  __shared__ uint8_t codes[4][128], signs[4][128];     // [wavefront][group 0: 0..31 | group 1: 32..127]
  for (int i = threadIdx.x; i < AKV_HYB_TABLE_FLOATS; i += 256) tab[i] = a.table[i];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const h25_roles r(lane);
  const float had_a = tab[H25_HAD + r.ca], had_b = tab[H25_HAD + r.cb];
  const float qjl_a = tab[H25_QJL + r.ca], qjl_b = tab[H25_QJL + r.cb];
  const float root_b = r.b0 ? kH25Root0 : kH25Root1;
  const int64_t n_total = (PAGED && a.x2) ? 2 * a.n : a.n;
  for (int64_t nn = (int64_t)blockIdx.x * 4 + wave; nn < n_total; nn += (int64_t)gridDim.x * 4) {
    const bool second = PAGED && nn >= a.n;                     // (wavefront-uniform)
    const int64_t n = second ? nn - a.n : nn;
    const void* xsrc = second ? a.x2 : a.x;
    const int64_t off = PAGED ? (n / a.heads) * a.xs0 + (n % a.heads) * a.xs1 : n * a.xs0;
    const float xa = akv_elem<XDT>::load(xsrc, off + r.ca);
    const float xb = akv_elem<XDT>::load(xsrc, off + r.cb);
    // norms: group 0 = the lower half's second values, group 1 = all first values + the upper half's second values
    const float sb = h25_half_sum(akv_mul_rn(xb, xb));
    const float n0 = sqrtf(h25_lane_value(sb, 0));
    const float n1 = sqrtf(akv_add_rn(akv_wave_sum(akv_mul_rn(xa, xa)), h25_lane_value(sb, 32)));
    const float ua = __fdiv_rn(xa, akv_add_rn(n1, 1e-10f));
    const float ub = __fdiv_rn(xb, akv_add_rn(r.b0 ? n0 : n1, 1e-10f));
    const float rot_a = __fdiv_rn(hyb_fwht64(akv_mul_rn(ua, had_a), lane), kH25Root1);
    const float rot_b = __fdiv_rn(h25_fwht32(akv_mul_rn(ub, had_b), lane), root_b);
    const uint32_t code_a = akv_search<1>(rot_a, tab + H25_BND1);
    const uint32_t code_b = r.b0 ? akv_search<2>(rot_b, tab + H25_BND0) : akv_search<1>(rot_b, tab + H25_BND1);
    const float cen_a = tab[H25_CEN1 + code_a];
    const float cen_b = r.b0 ? tab[H25_CEN0 + code_b] : tab[H25_CEN1 + code_b];
    const float mse_a = __fdiv_rn(akv_mul_rn(hyb_fwht64(cen_a, lane), had_a), kH25Root1);
    const float mse_b = __fdiv_rn(akv_mul_rn(h25_fwht32(cen_b, lane), had_b), root_b);
    const float res_a = akv_sub_rn(ua, mse_a), res_b = akv_sub_rn(ub, mse_b);
    const float rb = h25_half_sum(akv_mul_rn(res_b, res_b));
    const float rn0 = sqrtf(h25_lane_value(rb, 0));
    const float rn1 = sqrtf(akv_add_rn(akv_wave_sum(akv_mul_rn(res_a, res_a)), h25_lane_value(rb, 32)));
    const float proj_a = __fdiv_rn(hyb_fwht64(akv_mul_rn(res_a, qjl_a), lane), kH25Root1);
    const float proj_b = __fdiv_rn(h25_fwht32(akv_mul_rn(res_b, qjl_b), lane), root_b);
    codes[wave][r.ca] = (uint8_t)code_a;
    codes[wave][r.cb] = (uint8_t)code_b;
    signs[wave][r.ca] = proj_a >= 0.f ? 1 : 0;
    signs[wave][r.cb] = proj_b >= 0.f ? 1 : 0;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // lane k < 44 makes byte k of the row
    uint32_t byte = 0;
    const uint8_t* cw = codes[wave];
    const uint8_t* sw = signs[wave];
    if (lane < 8) byte = akv_stream_byte<2>(lane, [&](int d) { return (uint32_t)cw[d]; });
    else if (lane < 12) byte = akv_stream_byte<1>(lane - 8, [&](int d) { return (uint32_t)sw[d]; });
    else if (lane < 16) {
      const uint32_t hb = __half_as_ushort(__float2half_rn(lane < 14 ? n0 : rn0));
      byte = (lane & 1) ? hb >> 8 : hb & 0xffu;
    } else if (lane < 28) byte = akv_stream_byte<1>(lane - 16, [&](int d) { return (uint32_t)cw[32 + d]; });
    else if (lane < 40) byte = akv_stream_byte<1>(lane - 28, [&](int d) { return (uint32_t)sw[32 + d]; });
    else if (lane < 44) {
      const uint32_t hb = __half_as_ushort(__float2half_rn(lane < 42 ? n1 : rn1));
      byte = (lane & 1) ? hb >> 8 : hb & 0xffu;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
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
    if (lane < H25_ROW) dst[lane] = (uint8_t)byte;
  }
}

// ----------------------------------------------------------------------------------
// decode: one wavefront per vector
// ----------------------------------------------------------------------------------
// code, centroid and sign of the lane's two coordinates from a row in LDS or registers (byte accessor)
template <class F>
__device__ __forceinline__ void h25_row_values(const h25_roles& r, F byte_of, const float* cen0, const float* cen1,
                                               float& cen_a, float& sg_a, float& cen_b, float& sg_b) {
  cen_a = cen1[akv_stream_code<1>(r.ja, [&](int o) { return byte_of(16 + o); })];
  sg_a = ((byte_of(28 + (r.ja >> 3)) >> (7 - (r.ja & 7))) & 1u) ? 1.f : -1.f;
  if (r.b0) {
    cen_b = cen0[akv_stream_code<2>(r.jb, byte_of)];
    sg_b = ((byte_of(8 + (r.jb >> 3)) >> (7 - (r.jb & 7))) & 1u) ? 1.f : -1.f;
  } else {
    cen_b = cen1[akv_stream_code<1>(r.jb, [&](int o) { return byte_of(16 + o); })];
    sg_b = ((byte_of(28 + (r.jb >> 3)) >> (7 - (r.jb & 7))) & 1u) ? 1.f : -1.f;
  }
}

__global__ __launch_bounds__(256) void h25_decode_kernel(const uint8_t* __restrict__ packed, int64_t ps, int64_t n_vec,
                                                         const float* __restrict__ table, float* __restrict__ out,
                                                         int64_t os) {
  __shared__ float tab[AKV_HYB_TABLE_FLOATS];
  __shared__ uint8_t rows[4][64];
  for (int i = threadIdx.x; i < AKV_HYB_TABLE_FLOATS; i += 256) tab[i] = table[i];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const h25_roles r(lane);
  const float root_b = r.b0 ? kH25Root0 : kH25Root1;
  const float kappa_b = r.b0 ? kH25Kappa0 : kH25Kappa1;
  for (int64_t n = (int64_t)blockIdx.x * 4 + wave; n < n_vec; n += (int64_t)gridDim.x * 4) {
    if (lane < H25_ROW) rows[wave][lane] = packed[n * ps + lane];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const uint8_t* row = rows[wave];
    float cen_a, sg_a, cen_b, sg_b;
    h25_row_values(r, [&](int o) { return (uint32_t)row[o]; }, tab + H25_CEN0, tab + H25_CEN1, cen_a, sg_a, cen_b, sg_b);
    const float mse_a = __fdiv_rn(akv_mul_rn(hyb_fwht64(cen_a, lane), tab[H25_HAD + r.ca]), kH25Root1);
    const float mse_b = __fdiv_rn(akv_mul_rn(h25_fwht32(cen_b, lane), tab[H25_HAD + r.cb]), root_b);
    const float qjl_a = __fdiv_rn(akv_mul_rn(hyb_fwht64(sg_a * kH25Kappa1, lane), tab[H25_QJL + r.ca]), kH25Root1);
    const float qjl_b = __fdiv_rn(akv_mul_rn(h25_fwht32(sg_b * kappa_b, lane), tab[H25_QJL + r.cb]), root_b);
    const float n0 = h25_half_bits_to_float(row[12] | (row[13] << 8)), rn0 = h25_half_bits_to_float(row[14] | (row[15] << 8));
    const float n1 = h25_half_bits_to_float(row[40] | (row[41] << 8)), rn1 = h25_half_bits_to_float(row[42] | (row[43] << 8));
    out[n * os + r.ca] = akv_mul_rn(akv_add_rn(mse_a, akv_mul_rn(qjl_a, rn1)), n1);
    out[n * os + r.cb] = akv_mul_rn(akv_add_rn(mse_b, akv_mul_rn(qjl_b, r.b0 ? rn0 : rn1)), r.b0 ? n0 : n1);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// ----------------------------------------------------------------------------------
// attention
// ----------------------------------------------------------------------------------
struct h25_attn_args {
  const uint8_t* kc; int64_t kps_blk, kps_pos, kps_head;
  const uint8_t* vc; int64_t vps_blk, vps_pos, vps_head;
  const void* block_tables; int bt_itype; int64_t bt_stride;
  const void* context_lens; int cl_itype;
  const float* table;
  int S, QH, KVH, block_size;
  int64_t max_blocks_per_seq;
  int64_t num_blocks;  // physical blocks in the cache; table entries are clamped into [0, num_blocks)
  float scale;
  const int32_t* prefix;
  const float* qt;     // [S][QH][256]: Fwd_had(q) in coordinate order | kappa_g Fwd_qjl(q)
  float* part_acc;     // [G+S][QH][256]: sums in the Hadamard domain | sums in the QJL domain
  float* part_ml;
};

// prologue: 4 (sequence, query head) pairs per workgroup; the last workgroup does the prefix
template <int QDT>
__global__ __launch_bounds__(256) void h25_attn_prologue_kernel(
    const void* __restrict__ query, int64_t qs_seq, int64_t qs_head, const float* __restrict__ table,
    int S, int QH, const void* context_lens, int cl_itype, int block_size,
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
  const h25_roles r(lane);
  const int s = pair / QH, h = pair % QH;
  const int64_t off = s * qs_seq + h * qs_head;
  const float qa = akv_elem<QDT>::load(query, off + r.ca);
  const float qb = akv_elem<QDT>::load(query, off + r.cb);
  const float inv_b = r.b0 ? 1.f / kH25Root0 : 1.f / kH25Root1;
  const float kappa_b = r.b0 ? kH25Kappa0 : kH25Kappa1;
  float* o = qt + (size_t)pair * 256;
  o[r.ca] = hyb_fwht64(qa * table[H25_HAD + r.ca], lane) * (1.f / kH25Root1);
  o[r.cb] = h25_fwht32(qb * table[H25_HAD + r.cb], lane) * inv_b;
  o[128 + r.ca] = hyb_fwht64(qa * table[H25_QJL + r.ca], lane) * (1.f / kH25Root1) * kH25Kappa1;
  o[128 + r.cb] = h25_fwht32(qb * table[H25_QJL + r.cb], lane) * inv_b * kappa_b;
}

#define H25_WAVES 8
#define H25_VDW 11       // dwords of a row
#define H25_LUT_POS 144  // two-bit fields of a row's code and sign bytes (9 dwords x 16)

typedef uint32_t h25_u4 __attribute__((ext_vector_type(4)));
typedef float h25_f4 __attribute__((ext_vector_type(4)));
template <int GQ>
struct alignas(GQ * 4) h25_qv { float v[GQ]; };

// LDS of one wavefront, in floats:
//   lut [144][4][GQ]   partial dot products of the GQ query heads with the coordinates a two-bit field of a key
//                      row covers, for each of its four values (a 2-bit code: one coordinate of group 0; two
//                      1-bit codes or two sign bits: two coordinates)
//   p   [GQ][4][64]    weights of the chunk's tokens: p vn0 | p vn0 vr0 kappa0 | p vn1 | p vn1 vr1 kappa1
//   v   [11][64]       the chunk's value rows, dword-major (token = lane)
template <int GQ>
struct h25_attn_cfg {
  static constexpr size_t lut_floats = (size_t)H25_LUT_POS * 4 * GQ;
  static constexpr size_t wave_floats = lut_floats + 64 * GQ * 4 + 64 * H25_VDW;
  static size_t lds_bytes(int) { return (H25_WAVES * wave_floats + 8) * 4; }
};

template <int GQ>
__global__ __launch_bounds__(512) void h25_attn_kernel(h25_attn_args a) {
  typedef h25_attn_cfg<GQ> cfg;
  typedef h25_qv<GQ> qv;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  float* wave_base = (float*)lds_raw;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  qv* lut = (qv*)(wave_base + wave * cfg::wave_floats);
  float* p_lds = wave_base + wave * cfg::wave_floats + cfg::lut_floats;
  uint32_t* v_lds = (uint32_t*)(p_lds + 64 * GQ * 4);
  float cen0[4], cen1[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) cen0[i] = a.table[H25_CEN0 + i];
  cen1[0] = a.table[H25_CEN1]; cen1[1] = a.table[H25_CEN1 + 1];
  const h25_roles r(lane);

  // value phase, lane = coordinate pair: where the lane's bits sit in a row (dword, shift) and what they mean
  const int sh_a = 8 * ((lane >> 3) & 3) + 7 - (lane & 7);
  const int dw_a = 4 + (lane >> 5);                 // group-1 code dword; its sign dword is 3 further
  const int jb = 32 + lane;                         // lanes 32..63: position of the second coordinate in group 1
  const int dw_bm = r.b0 ? (lane >> 4) : 6;
  const int sh_bm = r.b0 ? 8 * ((lane >> 2) & 3) + 6 - 2 * (lane & 3) : 8 * ((jb >> 3) & 3) + 7 - (jb & 7);
  const int dw_bs = r.b0 ? 2 : 9;
  const int sh_bs = r.b0 ? 8 * (lane >> 3) + 7 - (lane & 7) : sh_bm;
  const float tb0 = r.b0 ? cen0[0] : cen1[0], tb1 = r.b0 ? cen0[1] : cen1[1];
  const float tb2 = r.b0 ? cen0[2] : cen1[0], tb3 = r.b0 ? cen0[3] : cen1[1];
  const int kb_m = r.b0 ? 0 : 2, kb_s = r.b0 ? 1 : 3;
  const uint32_t c1lo = __float_as_uint(cen1[0]), c1hi = __float_as_uint(cen1[1]);
  const uint32_t ub0 = __float_as_uint(tb0), ub1 = __float_as_uint(tb1), ub2 = __float_as_uint(tb2), ub3 = __float_as_uint(tb3);

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

    for (int h = wave; h < a.KVH; h += H25_WAVES) {
      for (int qg = 0; qg < gqa; qg += GQ) {
        // ---- table of the group's query heads (the wavefront's previous look-ups are done: LDS is in order)
        {
          const float* Q = a.qt + ((size_t)s * a.QH + (h * gqa + qg)) * 256;
          for (int e = lane; e < H25_LUT_POS * 4; e += 64) {
            const int pos = e >> 2, v = e & 3;
            const int di = pos >> 4, b = (pos >> 2) & 3, k = pos & 3;
            qv o;
            if (di < 2) {
#pragma unroll
              for (int q = 0; q < GQ; ++q) o.v[q] = Q[q * 256 + pos] * cen0[v];
            } else {
              const bool sign = di == 2 || di >= 6;
              const int base = di == 2 ? 128 : (di < 6 ? 32 : 160);
              const int ob = di == 2 ? b : 4 * ((di - 3) % 3) + b;
              const int j0 = base + 8 * ob + 2 * k;
              const float f_hi = sign ? ((v & 2) ? 1.f : -1.f) : cen1[v >> 1];
              const float f_lo = sign ? ((v & 1) ? 1.f : -1.f) : cen1[v & 1];
#pragma unroll
              for (int q = 0; q < GQ; ++q) o.v[q] = fmaf(Q[q * 256 + j0], f_hi, Q[q * 256 + j0 + 1] * f_lo);
            }
            lut[e] = o;
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        float m[GQ], l[GQ], acc[GQ][4];
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          m[q] = -INFINITY; l[q] = 0.f;
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[q][i] = 0.f;
        }

        for (int c0 = t0; c0 < t1; c0 += 64) {
          const int t = c0 + lane;
          const bool valid = t < t1;
          const int tc = valid ? t : t1 - 1;
          const int64_t phys = akv_clamp_block(akv_load_index(a.block_tables, a.bt_itype, s * a.bt_stride + tc / bs), a.num_blocks);
          const int pos = tc % bs;
          // ---- scores: lane = token, its key row in registers, one look-up per two-bit field
          uint32_t row[H25_VDW], vrow[H25_VDW];
          {
            const uint32_t* kr = (const uint32_t*)(a.kc + phys * a.kps_blk + pos * a.kps_pos + h * a.kps_head);
            const uint32_t* vr = (const uint32_t*)(a.vc + phys * a.vps_blk + pos * a.vps_pos + h * a.vps_head);
#pragma unroll
            for (int i = 0; i < H25_VDW; ++i) row[i] = kr[i];
#pragma unroll
            for (int i = 0; i < H25_VDW; ++i) vrow[i] = vr[i];
          }
          float d0[GQ], e0[GQ], d1[GQ], e1[GQ];
#pragma unroll
          for (int q = 0; q < GQ; ++q) { d0[q] = e0[q] = d1[q] = e1[q] = 0.f; }
#pragma unroll
          for (int di = 0; di < 9; ++di) {
            const uint32_t w = row[di < 3 ? di : di + 1];
#pragma unroll
            for (int c = 0; c < 16; ++c) {
              const uint32_t v = (w >> (8 * (c >> 2) + 6 - 2 * (c & 3))) & 3u;
              const qv e = lut[(16 * di + c) * 4 + v];
#pragma unroll
              for (int q = 0; q < GQ; ++q) {
                if (di < 2) d0[q] += e.v[q];
                else if (di == 2) e0[q] += e.v[q];
                else if (di < 6) d1[q] += e.v[q];
                else e1[q] += e.v[q];
              }
            }
          }
          const float kn0 = h25_half_bits_to_float(row[3]), kr0 = h25_half_bits_to_float(row[3] >> 16);
          const float kn1 = h25_half_bits_to_float(row[10]), kr1 = h25_half_bits_to_float(row[10] >> 16);
          // ---- value rows go to LDS dword-major; their norms stay here
#pragma unroll
          for (int i = 0; i < H25_VDW; ++i) v_lds[i * 64 + lane] = vrow[i];
          const float vn0 = h25_half_bits_to_float(vrow[3]), vr0 = h25_half_bits_to_float(vrow[3] >> 16);
          const float vn1 = h25_half_bits_to_float(vrow[10]), vr1 = h25_half_bits_to_float(vrow[10] >> 16);
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
            float* pw = p_lds + q * 256 + lane;
            pw[0] = valid ? p * vn0 : 0.f;
            pw[64] = valid ? p * vn0 * vr0 * kH25Kappa0 : 0.f;
            pw[128] = valid ? p * vn1 : 0.f;
            pw[192] = valid ? p * vn1 * vr1 * kH25Kappa1 : 0.f;
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          // ---- value sums: lane = coordinate pair, four tokens per read (the weights of tokens past the end are zero)
          const int nt = min(64, t1 - c0);
          for (int t4 = 0; t4 < nt; t4 += 4) {
            const h25_u4 wam = *(const h25_u4*)(v_lds + dw_a * 64 + t4);
            const h25_u4 was = *(const h25_u4*)(v_lds + (dw_a + 3) * 64 + t4);
            const h25_u4 wbm = *(const h25_u4*)(v_lds + dw_bm * 64 + t4);
            const h25_u4 wbs = *(const h25_u4*)(v_lds + dw_bs * 64 + t4);
            float cen_a[4], nsg_a[4], cen_b[4], nsg_b[4];     // nsg = -sign: bit set -> -1
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const uint32_t xam = wam[i], xas = was[i], xbm = wbm[i], xbs = wbs[i];
              // a bit as a mask of 32 (one signed bit-field extract), values picked by bitwise select
              const uint32_t ma = (uint32_t)__builtin_amdgcn_sbfe((int)xam, sh_a, 1);
              cen_a[i] = __uint_as_float((c1hi & ma) | (c1lo & ~ma));
              nsg_a[i] = __uint_as_float(((uint32_t)__builtin_amdgcn_sbfe((int)xas, sh_a, 1) & 0x80000000u) | 0x3f800000u);
              // lanes of group 1 have tb2 = tb0 and tb3 = tb1: whatever sits in the bit above their code changes nothing
              const uint32_t m0 = (uint32_t)__builtin_amdgcn_sbfe((int)xbm, sh_bm, 1);
              const uint32_t m1 = (uint32_t)__builtin_amdgcn_sbfe((int)xbm, sh_bm + 1, 1);
              const uint32_t lo = (ub1 & m0) | (ub0 & ~m0), hi = (ub3 & m0) | (ub2 & ~m0);
              cen_b[i] = __uint_as_float((hi & m1) | (lo & ~m1));
              nsg_b[i] = __uint_as_float(((uint32_t)__builtin_amdgcn_sbfe((int)xbs, sh_bs, 1) & 0x80000000u) | 0x3f800000u);
            }
#pragma unroll
            for (int q = 0; q < GQ; ++q) {
              const float* pq = p_lds + q * 256 + t4;
              const h25_f4 pz = *(const h25_f4*)(pq + 128), pw = *(const h25_f4*)(pq + 192);
              const h25_f4 pbm = *(const h25_f4*)(pq + kb_m * 64), pbs = *(const h25_f4*)(pq + kb_s * 64);
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const float z = pz[i], w = pw[i], bm = pbm[i], bsw = pbs[i];
                acc[q][0] = fmaf(z, cen_a[i], acc[q][0]);
                acc[q][1] = fmaf(-w, nsg_a[i], acc[q][1]);
                acc[q][2] = fmaf(bm, cen_b[i], acc[q][2]);
                acc[q][3] = fmaf(-bsw, nsg_b[i], acc[q][3]);
              }
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
          float* pa = a.part_acc + slot * 256;
          pa[r.ca] = acc[q][0]; pa[128 + r.ca] = acc[q][1];
          pa[r.cb] = acc[q][2]; pa[128 + r.cb] = acc[q][3];
          if (lane == 0) { a.part_ml[slot * 2] = m[q]; a.part_ml[slot * 2 + 1] = lsum; }
        }
      }
    }
  }
}

template <int ODT>
__global__ __launch_bounds__(64) void h25_attn_reduce_kernel(
    const int32_t* __restrict__ prefix, const float* __restrict__ part_acc,
    const float* __restrict__ part_ml, const float* __restrict__ table, int S, int QH, int G,
    void* __restrict__ out, int64_t os_seq, int64_t os_head, const uint32_t* __restrict__ status) {
  const int s = blockIdx.x / QH, h = blockIdx.x % QH;
  const int lane = threadIdx.x;
  const h25_roles r(lane);
  const int b0 = prefix[s], b1 = prefix[s + 1];
  const int64_t obase = s * os_seq + h * os_head;
  const float poison = status[0] != 0u ? __uint_as_float(0x7fc00000u) : 0.f;
  if (b1 <= b0) {
    akv_elem<ODT>::store(out, obase + r.ca, poison);
    akv_elem<ODT>::store(out, obase + r.cb, poison);
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
    const float* pa = part_acc + slot * 256;
    acc[0] = alpha * acc[0] + beta * pa[r.ca];
    acc[1] = alpha * acc[1] + beta * pa[128 + r.ca];
    acc[2] = alpha * acc[2] + beta * pa[r.cb];
    acc[3] = alpha * acc[3] + beta * pa[128 + r.cb];
  }
  const float inv = l > 0.f ? 1.f / l : 1.f;
  const float inv_b = r.b0 ? 1.f / kH25Root0 : 1.f / kH25Root1;
  const float oa = (hyb_fwht64(acc[0] * inv, lane) * table[H25_HAD + r.ca] +
                    hyb_fwht64(acc[1] * inv, lane) * table[H25_QJL + r.ca]) * (1.f / kH25Root1);
  const float ob = (h25_fwht32(acc[2] * inv, lane) * table[H25_HAD + r.cb] +
                    h25_fwht32(acc[3] * inv, lane) * table[H25_QJL + r.cb]) * inv_b;
  akv_elem<ODT>::store(out, obase + r.ca, oa + poison);
  akv_elem<ODT>::store(out, obase + r.cb, ob + poison);
}

// ----------------------------------------------------------------------------------
// host entries
// ----------------------------------------------------------------------------------
static int h25_grid(int64_t n) {
  int cus = akv_cached_cu_count();
  int64_t cap = (int64_t)(cus > 0 ? cus : 256) * 8;
  int64_t g = (n + 3) / 4;
  return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

template <bool PAGED>
static int h25_launch_encode(int dt, const h25_enc_args& a, hipStream_t stream) {
  const int grid = h25_grid((PAGED && a.x2) ? 2 * a.n : a.n);
  switch (dt) {
    case AKV_F16: h25_encode_kernel<AKV_F16, PAGED><<<grid, 256, 0, stream>>>(a); break;
    case AKV_BF16: h25_encode_kernel<AKV_BF16, PAGED><<<grid, 256, 0, stream>>>(a); break;
    default: h25_encode_kernel<AKV_F32, PAGED><<<grid, 256, 0, stream>>>(a); break;
  }
  AKV_LAUNCH_CHECK("h25_encode_kernel");
  return AKV_OK;
}

extern "C" int akv_hybrid25_encode(const void* x, int x_dtype, int64_t n, int64_t x_stride,
                                   const float* hyb_table, uint8_t* out, int64_t out_stride_bytes,
                                   void* stream) {
  AKV_REQUIRE(n >= 0 && akv_valid_dtype(x_dtype), "akv_hybrid25_encode: bad n / dtype");
  if (n == 0) return AKV_OK;
  AKV_REQUIRE(x && hyb_table && out, "akv_hybrid25_encode: null pointer");
  AKV_REQUIRE(x_stride >= 128 && out_stride_bytes >= H25_ROW, "akv_hybrid25_encode: stride smaller than row");
  h25_enc_args a = {};
  a.x = x; a.n = n; a.xs0 = x_stride; a.heads = 1; a.table = hyb_table;
  a.out = out; a.ps0 = out_stride_bytes;
  return h25_launch_encode<false>(x_dtype, a, (hipStream_t)stream);
}

extern "C" int akv_hybrid25_encode_paged(const void* x, int x_dtype, int64_t num_tokens,
                                         int num_kv_heads, int64_t xs_token, int64_t xs_head,
                                         const void* slot_mapping, int slot_itype,
                                         const float* hyb_table, uint8_t* out, int64_t ps_blk,
                                         int64_t ps_pos, int64_t ps_head, int block_size,
                                         int64_t max_blocks, void* stream) {
  AKV_REQUIRE(num_tokens >= 0 && num_kv_heads > 0, "akv_hybrid25_encode_paged: bad sizes");
  AKV_REQUIRE(akv_valid_dtype(x_dtype) && akv_valid_itype(slot_itype), "akv_hybrid25_encode_paged: bad dtype");
  AKV_REQUIRE(block_size > 0 && max_blocks >= 0, "akv_hybrid25_encode_paged: bad block_size/max_blocks");
  if (num_tokens == 0 || max_blocks == 0) return AKV_OK;
  AKV_REQUIRE(x && slot_mapping && hyb_table && out, "akv_hybrid25_encode_paged: null pointer");
  h25_enc_args a = {};
  a.x = x; a.n = num_tokens * num_kv_heads; a.xs0 = xs_token; a.xs1 = xs_head; a.heads = num_kv_heads;
  a.slots = slot_mapping; a.slot_itype = slot_itype; a.block_size = block_size; a.max_blocks = max_blocks;
  a.table = hyb_table; a.out = out; a.ps0 = ps_blk; a.ps1 = ps_pos; a.ps2 = ps_head;
  return h25_launch_encode<true>(x_dtype, a, (hipStream_t)stream);
}

extern "C" int akv_hybrid25_encode_paged_kv(const void* x_k, const void* x_v, int x_dtype, int64_t num_tokens,
                                            int num_kv_heads, int64_t xs_token, int64_t xs_head,
                                            const void* slot_mapping, int slot_itype,
                                            const float* hyb_table, uint8_t* out_k, uint8_t* out_v, int64_t ps_blk,
                                            int64_t ps_pos, int64_t ps_head, int block_size,
                                            int64_t max_blocks, void* stream) {
  AKV_REQUIRE(num_tokens >= 0 && num_kv_heads > 0, "akv_hybrid25_encode_paged_kv: bad sizes");
  AKV_REQUIRE(akv_valid_dtype(x_dtype) && akv_valid_itype(slot_itype), "akv_hybrid25_encode_paged_kv: bad dtype");
  AKV_REQUIRE(block_size > 0 && max_blocks >= 0, "akv_hybrid25_encode_paged_kv: bad block_size/max_blocks");
  if (num_tokens == 0 || max_blocks == 0) return AKV_OK;
  AKV_REQUIRE(x_k && x_v && slot_mapping && hyb_table && out_k && out_v, "akv_hybrid25_encode_paged_kv: null pointer");
  h25_enc_args a = {};
  a.x = x_k; a.x2 = x_v; a.n = num_tokens * num_kv_heads; a.xs0 = xs_token; a.xs1 = xs_head; a.heads = num_kv_heads;
  a.slots = slot_mapping; a.slot_itype = slot_itype; a.block_size = block_size; a.max_blocks = max_blocks;
  a.table = hyb_table; a.out = out_k; a.out2 = out_v; a.ps0 = ps_blk; a.ps1 = ps_pos; a.ps2 = ps_head;
  return h25_launch_encode<true>(x_dtype, a, (hipStream_t)stream);
}

extern "C" int akv_hybrid25_decode(const uint8_t* packed, int64_t packed_stride_bytes, int64_t n,
                                   const float* hyb_table, float* out, int64_t out_stride,
                                   void* stream) {
  AKV_REQUIRE(n >= 0, "akv_hybrid25_decode: n=%lld", (long long)n);
  if (n == 0) return AKV_OK;
  AKV_REQUIRE(packed && hyb_table && out, "akv_hybrid25_decode: null pointer");
  AKV_REQUIRE(packed_stride_bytes >= H25_ROW && out_stride >= 128, "akv_hybrid25_decode: stride smaller than row");
  h25_decode_kernel<<<h25_grid(n), 256, 0, (hipStream_t)stream>>>(packed, packed_stride_bytes, n, hyb_table, out, out_stride);
  AKV_LAUNCH_CHECK("h25_decode_kernel");
  return AKV_OK;
}

template <int GQ>
static int h25_launch_attn(const h25_attn_args& a, int grid, hipStream_t stream) {
  const size_t lds = h25_attn_cfg<GQ>::lds_bytes(a.QH);
  if (lds > 160 * 1024)
    return akv_fail(AKV_ERR_UNSUPPORTED, "hybrid25_paged_attn: too many query heads for LDS (%zu bytes)", lds);
  AKV_HIP(hipFuncSetAttribute((const void*)h25_attn_kernel<GQ>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  akv_profile_mark_begin(stream);
  h25_attn_kernel<GQ><<<grid, 512, lds, stream>>>(a);
  akv_profile_mark_end(stream);
  AKV_LAUNCH_CHECK("h25_attn_kernel");
  return AKV_OK;
}

extern "C" int akv_hybrid25_paged_attn(
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
  AKV_REQUIRE(num_seqs >= 0 && num_q_heads > 0 && num_kv_heads > 0, "akv_hybrid25_paged_attn: bad head/seq counts");
  AKV_REQUIRE((num_blocks > 0 && num_blocks < ((int64_t)1 << 31)) || max_blocks_per_seq == 0,
              "akv_hybrid25_paged_attn: num_blocks=%lld with a non-empty block table", (long long)num_blocks);
  AKV_REQUIRE(num_q_heads % num_kv_heads == 0, "akv_hybrid25_paged_attn: num_q_heads %% num_kv_heads != 0");
  AKV_REQUIRE(akv_valid_dtype(q_dtype) && akv_valid_dtype(out_dtype), "akv_hybrid25_paged_attn: bad dtype");
  AKV_REQUIRE(akv_valid_itype(bt_itype) && akv_valid_itype(cl_itype), "akv_hybrid25_paged_attn: bad index type");
  AKV_REQUIRE(block_size > 0 && max_blocks_per_seq >= 0, "akv_hybrid25_paged_attn: bad block_size / table width");
  if (num_seqs == 0) return AKV_OK;
  AKV_REQUIRE(query && out && hyb_table && context_lens, "akv_hybrid25_paged_attn: null pointer");
  AKV_REQUIRE(max_blocks_per_seq == 0 || (k_cache && v_cache && block_tables), "akv_hybrid25_paged_attn: null cache pointer");
  AKV_REQUIRE((((uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)kps_blk | (uintptr_t)kps_pos |
                (uintptr_t)kps_head | (uintptr_t)vps_blk | (uintptr_t)vps_pos | (uintptr_t)vps_head) & 3) == 0,
              "akv_hybrid25_paged_attn: packed rows must be 4-byte aligned");
  const int G = akv_attn_grid();
  AKV_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0, "akv_hybrid25_paged_attn: workspace null or not 256-byte aligned");
  akv_attn_ws ws = akv_attn_ws_layout(workspace, num_seqs, num_q_heads, 256, G);
  if (workspace_bytes < ws.bytes)
    return akv_fail(AKV_ERR_WORKSPACE, "akv_hybrid25_paged_attn: workspace %zu < %zu bytes", workspace_bytes, ws.bytes);

  const int nblocks_q = (num_seqs * num_q_heads + 3) / 4;
#define H25_PRO(DT) h25_attn_prologue_kernel<DT><<<nblocks_q + 1, 256, 0, stream>>>(query, qs_seq, qs_head, hyb_table, num_seqs, num_q_heads, context_lens, cl_itype, block_size, max_blocks_per_seq, ws.prefix, ws.qrot, nblocks_q, ws.status)
  if (q_dtype == AKV_F16) H25_PRO(AKV_F16); else if (q_dtype == AKV_BF16) H25_PRO(AKV_BF16); else H25_PRO(AKV_F32);
#undef H25_PRO
  AKV_LAUNCH_CHECK("h25_attn_prologue_kernel");

  h25_attn_args a;
  a.kc = k_cache; a.kps_blk = kps_blk; a.kps_pos = kps_pos; a.kps_head = kps_head;
  a.vc = v_cache; a.vps_blk = vps_blk; a.vps_pos = vps_pos; a.vps_head = vps_head;
  a.block_tables = block_tables; a.bt_itype = bt_itype; a.bt_stride = bt_stride;
  a.context_lens = context_lens; a.cl_itype = cl_itype; a.table = hyb_table;
  a.S = num_seqs; a.QH = num_q_heads; a.KVH = num_kv_heads; a.block_size = block_size;
  a.max_blocks_per_seq = max_blocks_per_seq; a.num_blocks = num_blocks; a.scale = scale;
  a.prefix = ws.prefix; a.qt = ws.qrot; a.part_acc = ws.part_acc; a.part_ml = ws.part_ml;
  const int gqa = num_q_heads / num_kv_heads;
  int rc = (gqa % 4 == 0) ? h25_launch_attn<4>(a, G, stream) : h25_launch_attn<1>(a, G, stream);
  if (rc) return rc;
  const int rgrid = num_seqs * num_q_heads;
  switch (out_dtype) {
    case AKV_F16: h25_attn_reduce_kernel<AKV_F16><<<rgrid, 64, 0, stream>>>(ws.prefix, ws.part_acc, ws.part_ml, hyb_table, num_seqs, num_q_heads, G, out, os_seq, os_head, ws.status); break;
    case AKV_BF16: h25_attn_reduce_kernel<AKV_BF16><<<rgrid, 64, 0, stream>>>(ws.prefix, ws.part_acc, ws.part_ml, hyb_table, num_seqs, num_q_heads, G, out, os_seq, os_head, ws.status); break;
    default: h25_attn_reduce_kernel<AKV_F32><<<rgrid, 64, 0, stream>>>(ws.prefix, ws.part_acc, ws.part_ml, hyb_table, num_seqs, num_q_heads, G, out, os_seq, os_head, ws.status); break;
  }
  AKV_LAUNCH_CHECK("h25_attn_reduce_kernel");
  return AKV_OK;
}
