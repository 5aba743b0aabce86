// tq35 rows and tables: what the codec, the vector attention kernel and the matrix-core attention
// kernel share.
//
// Row of one (token, kv head), 64 bytes (aither_kvcache/hybrid_quantizer.py:92-123,771-779):
//   [0,24)  group-0 codes, 3 bits each, MSB-first stream        [24,32) group-0 QJL sign bits (bit 7 first)
//   [32,34) group-0 norm fp16 LE    [34,36) group-0 residual norm fp16 LE
//   [36,52) group-1 codes, 2 bits each                           [52,60) group-1 QJL sign bits
//   [60,62) group-1 norm            [62,64) group-1 residual norm
// Table of floats handed to every entry point: sign vectors of the two structured transforms per
// group, the two codebooks, their decision boundaries.
#pragma once
#include "akv_common.h"

#define HYB_HAD0 0
#define HYB_HAD1 64
#define HYB_QJL0 128
#define HYB_QJL1 192
#define HYB_CEN0 256
#define HYB_CEN1 264
#define HYB_BND0 268
#define HYB_BND1 275

// 64-point Walsh-Hadamard transform across the lanes of a wavefront
template <int H>
__device__ __forceinline__ float hyb_fwht_step(float v, int lane) {
  const float o = akv_lane_xor<H>(v);
  return (lane & H) ? akv_sub_rn(o, v) : akv_add_rn(v, o);
}
__device__ __forceinline__ float hyb_fwht64(float v, int lane) {
  v = hyb_fwht_step<1>(v, lane);
  v = hyb_fwht_step<2>(v, lane);
  v = hyb_fwht_step<4>(v, lane);
  v = hyb_fwht_step<8>(v, lane);
  v = hyb_fwht_step<16>(v, lane);
  v = hyb_fwht_step<32>(v, lane);
  return v;
}

// matrix-core attention on tq35 rows (akv_attn_mfma.hip)
struct akv_hyb_mfma_args {
  const uint8_t* kc; int64_t kps_blk, kps_pos, kps_head;
  const uint8_t* vc; int64_t vps_blk, vps_pos, vps_head;
  const void* block_tables; int bt_itype; int64_t bt_stride;
  const void* context_lens; int cl_itype;
  int S, QH, KVH, hgroup, block_size;      // KVH counts groups of four query heads; hgroup of them share a kv head's rows
  int64_t max_blocks_per_seq;
  int64_t num_blocks;          // physical blocks in the cache; table entries are clamped into [0, num_blocks)
  const int32_t* prefix;
  uint32_t* status;            // status words of the call (workspace header)
  int spin_limit;              // polls a hand-off wait makes before it gives up
  const uint32_t* lut;         // table block, MF_W_*
  const uint4* qop;            // [S][KVH][16 k-steps][64 lanes] half8
  float* part_acc;             // [G + S][QH][256]: A0 | B0 | A1 | B1, natural coordinate order
  float* part_ml;
  float kappa;                 // sqrt(pi/2)/64, applied to the sign sums
};

size_t akv_hyb_mfma_extra_bytes(int S, int QH);
bool akv_hyb_mfma_applicable(int QH, int KVH, int block_size, const int64_t* strides6);
int akv_hyb_mfma_run(const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head, const float* table, float kappa,
                     float scale, akv_hyb_mfma_args a, int block_size, int32_t* prefix, uint32_t* lut, void* extra_ws,
                     int grid, hipStream_t stream);
