// Block selection for sparse decode attention over a 4-bit TurboQuant cache
// (aither_kvcache/block_selector.py): per-block key representatives kept from the packed codes,
// block scores against the GQA-mean rotated query, and a fixed-size top-k of the table columns.
//
//   update    one workgroup per (new token, kv head): lane = code byte; the norm-weighted centroids
//             of its two nibbles go to the block's accumulators by float atomics (the order of
//             the additions is that of the hardware, as with the reference's scatter_add_ on a GPU)
//   finalize  rep = acc / max(count, 1) for the listed blocks (all when no list is given)
//   scores    one workgroup per (sequence, 64 table columns); the mean query of every GQA group is
//             formed once in LDS, a wavefront then takes 16 columns, one dot product of
//             2 x kv_heads x half_d terms each
//   select    one workgroup per sequence: an 8-bit radix select (four passes) finds the k-th largest
//             key and how many of the keys equal to it belong to the top k (lowest column first),
//             then the chosen columns are written in column order through two block-wide scans
#include "akv_common.h"

#define BS_THREADS 1024
#define BS_COLS 4            // table columns per wavefront of the scoring kernel

__global__ __launch_bounds__(64) void bs_update_kernel(const void* __restrict__ bidx, int itype, const uint8_t* __restrict__ kp,
                                                       int64_t ps_tok, int64_t ps_head, const float* __restrict__ kn,
                                                       int64_t ns_tok, int64_t ns_head, const float* __restrict__ centroids,
                                                       float* __restrict__ acc_e, float* __restrict__ acc_o,
                                                       int32_t* __restrict__ counts, int64_t max_blocks, int H, int PD) {
  const int64_t i = blockIdx.x / H;
  const int h = blockIdx.x % H;
  const int64_t b = akv_load_index(bidx, itype, i);
  if (b < 0 || b >= max_blocks) return;
  const float w = kn[i * ns_tok + h * ns_head];
  const uint8_t* row = kp + i * ps_tok + h * ps_head;
  float* ae = acc_e + ((size_t)b * H + h) * PD;
  float* ao = acc_o + ((size_t)b * H + h) * PD;
  for (int t = threadIdx.x; t < PD; t += 64) {
    const uint32_t byte = row[t];
    atomicAdd(ae + t, w * centroids[byte >> 4]);
    atomicAdd(ao + t, w * centroids[byte & 15u]);
  }
  if (threadIdx.x == 0) atomicAdd(counts + (size_t)b * H + h, 1);
}

// grid.x = listed blocks (or all blocks), one workgroup per block
__global__ __launch_bounds__(256) void bs_finalize_kernel(const void* __restrict__ bidx, int itype,
                                                          const float* __restrict__ acc_e, const float* __restrict__ acc_o,
                                                          const int32_t* __restrict__ counts, float* __restrict__ rep_e,
                                                          float* __restrict__ rep_o, int64_t max_blocks, int H, int PD) {
  const int64_t b = bidx ? akv_load_index(bidx, itype, blockIdx.x) : (int64_t)blockIdx.x;
  if (b < 0 || b >= max_blocks) return;
  for (int t = threadIdx.x; t < H * PD; t += 256) {
    const int c = counts[(size_t)b * H + t / PD];
    const float safe = (float)(c > 1 ? c : 1);
    const size_t o = (size_t)b * H * PD + t;
    rep_e[o] = acc_e[o] / safe;
    rep_o[o] = acc_o[o] / safe;
  }
}

__global__ __launch_bounds__(256) void bs_scores_kernel(const float* __restrict__ q_even, const float* __restrict__ q_odd,
                                                        const float* __restrict__ rep_e, const float* __restrict__ rep_o,
                                                        const void* __restrict__ bt, int bt_itype, int64_t bt_stride,
                                                        const void* __restrict__ cl, int cl_itype, int QH, int KVH, int HD,
                                                        int64_t B, int block_size, int64_t num_blocks, float* __restrict__ scores) {
  extern __shared__ float qm[];     // [2][KVH][HD]: mean even / odd query of each GQA group
  const int s = blockIdx.y;
  const int gqa = QH / KVH;
  const float inv = 1.0f / (float)gqa;
  for (int i = threadIdx.x; i < KVH * HD; i += 256) {
    const int kv = i / HD, d = i % HD;
    float se = 0.f, so = 0.f;
    for (int g = 0; g < gqa; ++g) {
      se += q_even[((size_t)s * QH + kv * gqa + g) * HD + d];
      so += q_odd[((size_t)s * QH + kv * gqa + g) * HD + d];
    }
    qm[i] = se * inv;
    qm[KVH * HD + i] = so * inv;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t ctx = akv_load_index(cl, cl_itype, s);
  const int64_t nb = (ctx + block_size - 1) / block_size;
  const int n = KVH * HD;
  // A wavefront takes BS_COLS columns at once: their table entries, then their representatives, are requested
  // together (one column after the other is a chain of two trips to memory per column -- 22 us for 128 columns of
  // 16 sequences); every column's sum is formed in the order it always was.
  const int64_t col0 = (int64_t)blockIdx.x * (4 * BS_COLS) + wave * BS_COLS;
  const float* re[BS_COLS];
  const float* ro[BS_COLS];
  bool live[BS_COLS];
#pragma unroll
  for (int j = 0; j < BS_COLS; ++j) {
    const int64_t col = col0 + j;
    live[j] = col < B && col < nb;
    int64_t blk = live[j] ? akv_load_index(bt, bt_itype, s * bt_stride + col) : 0;
    blk = blk < 0 ? 0 : (blk >= num_blocks ? num_blocks - 1 : blk);
    re[j] = rep_e + (size_t)blk * n;
    ro[j] = rep_o + (size_t)blk * n;
  }
  float acc[BS_COLS];
#pragma unroll
  for (int j = 0; j < BS_COLS; ++j) acc[j] = 0.f;
  for (int i = lane; i < n; i += 64) {
    const float qe = qm[i], qo = qm[n + i];
#pragma unroll
    for (int j = 0; j < BS_COLS; ++j)
      if (live[j]) acc[j] = fmaf(qe, re[j][i], fmaf(qo, ro[j][i], acc[j]));
  }
#pragma unroll
  for (int j = 0; j < BS_COLS; ++j) {
    const int64_t col = col0 + j;
    const float r = live[j] ? akv_wave_sum(acc[j]) : -INFINITY;
    if (lane == 0 && col < B) scores[(size_t)s * B + col] = r;
  }
}

// larger float <-> larger unsigned; the two zeros share a key (they compare equal, so the lower column wins
// between them like between any equal scores) and a NaN of either sign ranks above everything, +inf included,
// as torch.topk ranks it
__device__ __forceinline__ uint32_t bs_key(float v) {
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;
  if (u == 0x80000000u) u = 0u;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ uint32_t bs_column_key(const float* __restrict__ sc, int64_t col, int64_t nb, int sinks, int recents) {
  if (col >= nb) return bs_key(-INFINITY);
  if (col < sinks || col >= nb - recents) return bs_key(INFINITY);
  return bs_key(sc[col]);
}

// exclusive scan of one int per thread over the 1024 threads of the workgroup; also returns the total
__device__ __forceinline__ int bs_block_scan(int v, int* lds /*[17]*/, int& total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int inc = akv_wave_inclusive_scan(v);
  __syncthreads();
  if (lane == 63) lds[wave] = inc;
  __syncthreads();
  int base = 0, tot = 0;
  for (int w = 0; w < BS_THREADS / 64; ++w) {
    const int t = lds[w];
    if (w < wave) base += t;
    tot += t;
  }
  total = tot;
  return base + inc - v;
}

template <typename BT, typename CL>
__global__ __launch_bounds__(BS_THREADS) void bs_select_kernel(const float* __restrict__ scores, const BT* __restrict__ bt,
                                                               int64_t bt_stride, const CL* __restrict__ cl, int64_t B,
                                                               int block_size, int max_selected, int sinks, int recents,
                                                               BT* __restrict__ fbt, CL* __restrict__ fcl) {
  __shared__ int hist[256];
  __shared__ int scan_lds[17];
  __shared__ uint32_t sh_prefix;
  __shared__ int sh_krem;
  const int s = blockIdx.x;
  const float* sc = scores + (size_t)s * B;
  const int64_t ctx = (int64_t)cl[s];
  const int64_t nb = (ctx + block_size - 1) / block_size;
  const int k = (int)(max_selected < B ? max_selected : B);
  // ---- radix select: after the passes, `prefix` is the k-th largest key and `krem` the number of
  // columns holding exactly that key that belong to the top k
  uint32_t prefix = 0;
  int krem = k;
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    const uint32_t known = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
    for (int i = threadIdx.x; i < 256; i += BS_THREADS) hist[i] = 0;
    __syncthreads();
    for (int64_t col = threadIdx.x; col < B; col += BS_THREADS) {
      const uint32_t key = bs_column_key(sc, col, nb, sinks, recents);
      if ((key & known) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1);
    }
    __syncthreads();
    {
      // the highest bucket at which the count of keys in it and above reaches krem (bucket 0 if none does): thread
      // b < 256 knows how many keys lie above its bucket from a scan over the buckets, and exactly one thread finds
      // above < krem <= above + its own count.  (One thread walking down from bucket 255 read up to 255 counters
      // one after the other, four times: 25-50 us per call.)
      const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
      const int mine = threadIdx.x < 256 ? hist[threadIdx.x] : 0;
      const int inc = akv_wave_inclusive_scan(mine);
      if (threadIdx.x < 256 && lane == 63) scan_lds[wave] = inc;
      __syncthreads();
      if (threadIdx.x < 256) {
        int below_waves = 0, total = 0;
        for (int w = 0; w < 4; ++w) {
          const int t = scan_lds[w];
          if (w < wave) below_waves += t;
          total += t;
        }
        const int above = total - (below_waves + inc);       // keys in buckets above this one
        if (above < krem && (threadIdx.x == 0 || above + mine >= krem)) {
          sh_prefix = prefix | ((uint32_t)threadIdx.x << shift);
          sh_krem = krem - above;
        }
      }
    }
    __syncthreads();
    prefix = sh_prefix;
    krem = sh_krem;
    __syncthreads();
  }
  // ---- columns in order: thread t owns the contiguous columns [t * chunk, (t + 1) * chunk)
  const int64_t chunk = (B + BS_THREADS - 1) / BS_THREADS;
  const int64_t c0 = (int64_t)threadIdx.x * chunk, c1 = c0 + chunk < B ? c0 + chunk : B;
  int n_eq = 0, n_gt = 0;
  for (int64_t col = c0; col < c1; ++col) {
    const uint32_t key = bs_column_key(sc, col, nb, sinks, recents);
    n_eq += key == prefix ? 1 : 0;
    n_gt += key > prefix ? 1 : 0;
  }
  int tot;
  const int eq_before = bs_block_scan(n_eq, scan_lds, tot);
  int n_take = 0, eq_seen = eq_before;
  for (int64_t col = c0; col < c1; ++col)
    if (bs_column_key(sc, col, nb, sinks, recents) == prefix) n_take += (eq_seen++ < krem) ? 1 : 0;
  int out = bs_block_scan(n_gt + n_take, scan_lds, tot);
  eq_seen = eq_before;
  for (int64_t col = c0; col < c1; ++col) {
    const uint32_t key = bs_column_key(sc, col, nb, sinks, recents);
    const bool take = key > prefix || (key == prefix && eq_seen++ < krem);
    if (take) fbt[(size_t)s * max_selected + out++] = bt[s * bt_stride + col];
  }
  for (int j = k + threadIdx.x; j < max_selected; j += BS_THREADS) fbt[(size_t)s * max_selected + j] = (BT)0;
  if (threadIdx.x == 0) {
    const int64_t cap = (int64_t)k * block_size;
    fcl[s] = (CL)(ctx < cap ? ctx : cap);
  }
}

// ----------------------------------------------------------------------------------
// C ABI
// ----------------------------------------------------------------------------------
extern "C" int akv_block_rep_finalize(const void* block_indices, int idx_itype, int64_t n, const float* acc_even,
                                      const float* acc_odd, const int32_t* counts, float* rep_even, float* rep_odd,
                                      int64_t max_blocks, int num_kv_heads, int packed_dim, void* stream) {
  AKV_REQUIRE(max_blocks >= 0 && num_kv_heads > 0 && packed_dim > 0 && n >= 0, "akv_block_rep_finalize: bad sizes");
  AKV_REQUIRE(!block_indices || akv_valid_itype(idx_itype), "akv_block_rep_finalize: bad index type");
  const int64_t grid = block_indices ? n : max_blocks;
  if (grid == 0) return AKV_OK;
  AKV_REQUIRE(acc_even && acc_odd && counts && rep_even && rep_odd, "akv_block_rep_finalize: null pointer");
  AKV_REQUIRE(grid < ((int64_t)1 << 31), "akv_block_rep_finalize: too many blocks");
  bs_finalize_kernel<<<(int)grid, 256, 0, (hipStream_t)stream>>>(block_indices, idx_itype, acc_even, acc_odd, counts, rep_even,
                                                                rep_odd, max_blocks, num_kv_heads, packed_dim);
  AKV_LAUNCH_CHECK("bs_finalize_kernel");
  return AKV_OK;
}

extern "C" int akv_block_rep_update(const void* block_indices, int idx_itype, int64_t n, const uint8_t* k_packed,
                                    int64_t ps_tok, int64_t ps_head, const float* k_norms, int64_t ns_tok, int64_t ns_head,
                                    const float* centroids, float* acc_even, float* acc_odd, int32_t* counts, float* rep_even,
                                    float* rep_odd, int64_t max_blocks, int num_kv_heads, int packed_dim, void* stream) {
  AKV_REQUIRE(n >= 0 && max_blocks >= 0 && num_kv_heads > 0 && packed_dim > 0, "akv_block_rep_update: bad sizes");
  AKV_REQUIRE(akv_valid_itype(idx_itype), "akv_block_rep_update: bad index type");
  if (n == 0) return AKV_OK;
  AKV_REQUIRE(block_indices && k_packed && k_norms && centroids && acc_even && acc_odd && counts,
              "akv_block_rep_update: null pointer");
  AKV_REQUIRE((rep_even == nullptr) == (rep_odd == nullptr), "akv_block_rep_update: give both representative arrays or neither");
  AKV_REQUIRE(n * num_kv_heads < ((int64_t)1 << 31), "akv_block_rep_update: too many tokens");
  bs_update_kernel<<<(int)(n * num_kv_heads), 64, 0, (hipStream_t)stream>>>(block_indices, idx_itype, k_packed, ps_tok, ps_head,
                                                                            k_norms, ns_tok, ns_head, centroids, acc_even, acc_odd,
                                                                            counts, max_blocks, num_kv_heads, packed_dim);
  AKV_LAUNCH_CHECK("bs_update_kernel");
  if (!rep_even) return AKV_OK;
  // the blocks just touched (a block listed twice is finalised twice, to the same values)
  return akv_block_rep_finalize(block_indices, idx_itype, n, acc_even, acc_odd, counts, rep_even, rep_odd, max_blocks,
                                num_kv_heads, packed_dim, stream);
}

extern "C" int akv_block_scores(const float* q_even, const float* q_odd, const float* rep_even, const float* rep_odd,
                                const void* block_tables, int bt_itype, int64_t bt_stride, const void* context_lens,
                                int cl_itype, int num_seqs, int num_q_heads, int num_kv_heads, int half_d,
                                int64_t max_blocks_per_seq, int block_size, int64_t num_blocks, float* scores, void* stream) {
  AKV_REQUIRE(num_seqs >= 0 && num_q_heads > 0 && num_kv_heads > 0 && half_d > 0, "akv_block_scores: bad sizes");
  AKV_REQUIRE(num_q_heads % num_kv_heads == 0, "akv_block_scores: num_q_heads %% num_kv_heads != 0");
  AKV_REQUIRE(max_blocks_per_seq >= 0 && block_size > 0 && num_blocks > 0, "akv_block_scores: bad block counts");
  AKV_REQUIRE(akv_valid_itype(bt_itype) && akv_valid_itype(cl_itype), "akv_block_scores: bad index type");
  if (num_seqs == 0 || max_blocks_per_seq == 0) return AKV_OK;
  AKV_REQUIRE(q_even && q_odd && rep_even && rep_odd && block_tables && context_lens && scores, "akv_block_scores: null pointer");
  const size_t lds = (size_t)2 * num_kv_heads * half_d * sizeof(float);
  if (lds > 48 * 1024) return akv_fail(AKV_ERR_UNSUPPORTED, "akv_block_scores: kv_heads x half_d = %d too large", num_kv_heads * half_d);
  const dim3 grid((unsigned)((max_blocks_per_seq + 4 * BS_COLS - 1) / (4 * BS_COLS)), (unsigned)num_seqs);
  bs_scores_kernel<<<grid, 256, lds, (hipStream_t)stream>>>(q_even, q_odd, rep_even, rep_odd, block_tables, bt_itype, bt_stride,
                                                           context_lens, cl_itype, num_q_heads, num_kv_heads, half_d,
                                                           max_blocks_per_seq, block_size, num_blocks, scores);
  AKV_LAUNCH_CHECK("bs_scores_kernel");
  return AKV_OK;
}

extern "C" int akv_block_select(const float* scores, const void* block_tables, int bt_itype, int64_t bt_stride,
                                const void* context_lens, int cl_itype, int num_seqs, int64_t max_blocks_per_seq,
                                int block_size, int max_selected, int num_sink_blocks, int num_recent_blocks,
                                void* filtered_block_tables, void* filtered_context_lens, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  AKV_REQUIRE(num_seqs >= 0 && max_blocks_per_seq > 0 && block_size > 0 && max_selected > 0, "akv_block_select: bad sizes");
  AKV_REQUIRE(num_sink_blocks >= 0 && num_recent_blocks >= 0, "akv_block_select: bad sink / recent counts");
  AKV_REQUIRE(akv_valid_itype(bt_itype) && akv_valid_itype(cl_itype), "akv_block_select: bad index type");
  if (num_seqs == 0) return AKV_OK;
  AKV_REQUIRE(scores && block_tables && context_lens && filtered_block_tables && filtered_context_lens,
              "akv_block_select: null pointer");
#define BS_LAUNCH(BT, CL)                                                                                             \
  bs_select_kernel<BT, CL><<<num_seqs, BS_THREADS, 0, stream>>>(scores, (const BT*)block_tables, bt_stride,          \
      (const CL*)context_lens, max_blocks_per_seq, block_size, max_selected, num_sink_blocks, num_recent_blocks,     \
      (BT*)filtered_block_tables, (CL*)filtered_context_lens)
  if (bt_itype == AKV_I64 && cl_itype == AKV_I64) BS_LAUNCH(int64_t, int64_t);
  else if (bt_itype == AKV_I64) BS_LAUNCH(int64_t, int32_t);
  else if (cl_itype == AKV_I64) BS_LAUNCH(int32_t, int64_t);
  else BS_LAUNCH(int32_t, int32_t);
#undef BS_LAUNCH
  AKV_LAUNCH_CHECK("bs_select_kernel");
  return AKV_OK;
}
