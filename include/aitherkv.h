/*
 * aitherkv.h -- C ABI of the MI355X (gfx950) TurboQuant KV-cache hot path.
 *
 * The reference (aither-kvcache) has no FFI of its own: its hot path is Python
 * calling torch ops and Triton kernels.  This header is the boundary a binding
 * for that path would use: plain device pointers, element strides, sizes, enums
 * and a hipStream_t; every function returns an akv_status and never aborts
 * (the reference's callers wrap the path in try/except and fall back,
 * aither_kvcache/vllm/backend.py:527-530,552-555).  Each entry point cites the
 * reference function it stands in for.
 *
 * Conventions
 *   - all pointers are DEVICE pointers unless said otherwise; the caller owns
 *     every buffer; nothing is allocated or freed by the library except where a
 *     function says so;
 *   - strides are in ELEMENTS of the pointed-to type unless the name ends in
 *     _bytes;
 *   - work is enqueued on `stream` (void* = hipStream_t; NULL = default stream)
 *     and the call returns without synchronising;
 *   - packed code layouts are the reference's: aither_kvcache/packing.py:13-118
 *     (4-bit: byte k = idx[2k]<<4 | idx[2k+1]; 2-bit: 4 per byte, first index in
 *     the top bits; 3-bit: 8 indices -> 24-bit big-endian word, index 0 in bits
 *     23..21) and aither_kvcache/hybrid_quantizer.py:92-123 for tq35.
 */
#ifndef AITHERKV_H
#define AITHERKV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  AKV_OK = 0,
  AKV_ERR_INVALID = 1,     /* bad argument (null pointer, negative size, bad enum) */
  AKV_ERR_UNSUPPORTED = 2, /* valid request this build has no kernel for          */
  AKV_ERR_WORKSPACE = 3,   /* workspace missing or too small                       */
  AKV_ERR_HIP = 4          /* a HIP runtime call failed; see akv_last_error()      */
} akv_status;

typedef enum { AKV_F16 = 0, AKV_BF16 = 1, AKV_F32 = 2 } akv_dtype;
typedef enum { AKV_I32 = 0, AKV_I64 = 1 } akv_itype;

/* Library version string (static storage). */
const char* akv_version(void);
/* Message for the last non-OK status returned on this host thread (static storage). */
const char* akv_last_error(void);
/* Number of compute units of the current device (0 and a status if no device). */
int akv_device_cu_count(int* cu_count);

/* ---------------------------------------------------------------------------------
 * Measurement hook (no counterpart in the reference).  While enabled, every entry point
 * times its dominant kernel (the main decode-attention kernel, the encode kernel, the
 * TriAttention scoring kernel) with a pair of HIP events on the launch stream: the matrix-core
 * kernels are launched with the pair attached to the dispatch (its own start and end time
 * stamps, as a kernel trace reports them), the others are bracketed by two recorded events.
 * The pairs go into a ring of 64, and nothing is read back between calls, so sampled calls
 * run back to back.  akv_profile_last_ms waits for the pair of the most recent call and
 * returns its elapsed time in milliseconds; akv_profile_mean_ms waits for the most recent
 * pair and returns the mean over the (at most 64) latest pairs recorded since the hook was
 * switched on, with their number in *samples (may be NULL).  Meant for benchmarks; leave
 * it off in serving code.
 * ------------------------------------------------------------------------------- */
int akv_profile_enable(int on);
int akv_profile_last_ms(float* ms);
int akv_profile_mean_ms(float* ms, int* samples);

/* ---------------------------------------------------------------------------------
 * Rotation matrix, prepared once per quantizer.
 * `rotation` is the reference's Pi (row-major [d,d] float32, y = Pi x,
 * aither_kvcache/rotation.py:20-35, used as x @ Pi.T at quantizer.py:150).  The
 * kernels want it in several layouts (Pi, Pi^T, and fp16 hi/lo MFMA tiles);
 * akv_rotation_prepare writes them all into `prep` (device, akv_rotation_prepared_bytes(d)
 * bytes, 256-byte aligned), which the entry points below take instead of `rotation`.
 * ------------------------------------------------------------------------------- */
size_t akv_rotation_prepared_bytes(int d);
int akv_rotation_prepare(const float* rotation, int d, void* prep, size_t prep_bytes, void* stream);

/* ---------------------------------------------------------------------------------
 * Codec primitives -- aither_kvcache/triton_ops.py:220-259
 * (triton_quantize_4bit/2bit, triton_dequantize_4bit/2bit; 3-bit is a stub there and
 * real here).  Ties follow the torch path (quantizer.py:203-207): code = #{b : b < y}.
 * ------------------------------------------------------------------------------- */
int akv_quantize_pack(const float* y, int64_t n, int d, int64_t y_stride,
                      const float* boundaries, int bits,
                      uint8_t* out, int64_t out_stride, void* stream);
int akv_unpack_lookup(const uint8_t* packed, int64_t n, int d, int64_t packed_stride,
                      const float* centroids, int bits,
                      float* out, int64_t out_stride, void* stream);

/* ---------------------------------------------------------------------------------
 * TurboQuant.encode -- aither_kvcache/quantizer.py:122-166.
 * n vectors of d elements (row stride x_stride): norm, x/(norm+1e-10), rotation,
 * codebook search, packing.  Writes out_packed[n][packed_size(d,bits)] (row stride
 * packed_stride bytes) and out_norms[n] (float32).
 * ------------------------------------------------------------------------------- */
int akv_encode(const void* x, int x_dtype, int64_t n, int d, int64_t x_stride,
               const void* rot_prep, const float* boundaries, int bits,
               uint8_t* out_packed, int64_t packed_stride, float* out_norms, void* stream);

/* ---------------------------------------------------------------------------------
 * fused_tq4_kv_update -- aither_kvcache/fused_kv_update.py:300-405 (semantics of its
 * torch fallback :220-293), for 4-, 3- and 2-bit.
 * x[num_tokens][num_kv_heads][d]; slot = slot_mapping[token]; tokens with slot < 0 or
 * slot / block_size >= max_blocks are skipped; writes
 *   out_packed[blk*ps_blk + pos*ps_pos + head*ps_head + 0..packed)   (uint8)
 *   out_norms [blk*ns_blk + pos*ns_pos + head*ns_head]               (float32)
 * ------------------------------------------------------------------------------- */
int akv_encode_paged(const void* x, int x_dtype, int64_t num_tokens, int num_kv_heads, int d,
                     int64_t xs_token, int64_t xs_head,
                     const void* slot_mapping, int slot_itype,
                     const void* rot_prep, const float* boundaries, int bits,
                     uint8_t* out_packed, int64_t ps_blk, int64_t ps_pos, int64_t ps_head,
                     float* out_norms, int64_t ns_blk, int64_t ns_pos, int64_t ns_head,
                     int block_size, int64_t max_blocks, void* stream);

/* ---------------------------------------------------------------------------------
 * K and V of one serving step in ONE launch -- what fused_encode_and_store does with two
 * calls, aither_kvcache/fused_kv_update.py:412-468.  k and v are [num_tokens][num_kv_heads][d]
 * with the same strides and dtype; the two caches and the two norm tensors share their
 * strides as well (the K and V halves of one serving cache tensor do); one slot_mapping.
 * Same results as two akv_encode_paged calls.
 * ------------------------------------------------------------------------------- */
int akv_encode_paged_kv(const void* k, const void* v, int x_dtype, int64_t num_tokens,
                        int num_kv_heads, int d, int64_t xs_token, int64_t xs_head,
                        const void* slot_mapping, int slot_itype,
                        const void* rot_prep, const float* boundaries, int bits,
                        uint8_t* k_packed, uint8_t* v_packed,
                        int64_t ps_blk, int64_t ps_pos, int64_t ps_head,
                        float* k_norms, float* v_norms,
                        int64_t ns_blk, int64_t ns_pos, int64_t ns_head,
                        int block_size, int64_t max_blocks, void* stream);

/* ---------------------------------------------------------------------------------
 * TurboQuant.decode -- aither_kvcache/quantizer.py:168-197:
 * out[i] = (centroids[codes_i] @ Pi) * norms[i], cast to out_dtype.
 * ------------------------------------------------------------------------------- */
int akv_decode(const uint8_t* packed, int64_t packed_stride, const float* norms, int64_t n, int d,
               const void* rot_prep, const float* centroids, int bits,
               void* out, int out_dtype, int64_t out_stride, void* stream);

/* ---------------------------------------------------------------------------------
 * TurboQuantImpl._batch_decompress_active_blocks -- aither_kvcache/vllm/backend.py:1040-1091
 * (unique block ids -> gather packed rows and norms -> TurboQuant.decode -> scatter), as
 * one pass with no gather, unique or scatter step: for every i < num_ids whose
 * b = block_ids[i] lies in [0, num_blocks), all block_size * num_kv_heads rows of cache
 * block b are decoded into block b of `out`.  Ids outside the cache are skipped (the
 * reference filters them, :1063); an id listed twice writes the same values twice.
 *   packed  [num_blocks][block_size][num_kv_heads][>= packed bytes], byte strides ps_*
 *   norms   [num_blocks][block_size][num_kv_heads] float32, element strides ns_*
 *   out     [num_blocks][block_size][num_kv_heads][d], element strides os_*, last dim contiguous
 * block_ids may be the flattened block table itself (padding entries negative).
 * ------------------------------------------------------------------------------- */
int akv_decode_blocks(const uint8_t* packed, int64_t ps_blk, int64_t ps_pos, int64_t ps_head,
                      const float* norms, int64_t ns_blk, int64_t ns_pos, int64_t ns_head,
                      const void* block_ids, int ids_itype, int64_t num_ids, int64_t num_blocks,
                      int block_size, int num_kv_heads, int d,
                      const void* rot_prep, const float* centroids, int bits,
                      void* out, int out_dtype, int64_t os_blk, int64_t os_pos, int64_t os_head,
                      void* stream);

/* ---------------------------------------------------------------------------------
 * TQPagedAttention.forward -- aither_kvcache/fused_attention.py:594-748, with the result
 * of TQPagedAttentionRef.forward (:91-185).  The query pre-rotation (:659) and the output
 * inverse rotation (:747) are done inside.
 *   query        [num_seqs][num_q_heads][d], strides qs_seq / qs_head (last dim contiguous)
 *   k/v_packed   [blocks][block_size][num_kv_heads][packed] uint8, strides in bytes
 *   k/v_norms    [blocks][block_size][num_kv_heads] float32, strides in elements
 *   block_tables [num_seqs][max_blocks_per_seq] (row stride bt_stride); entries at or
 *                beyond ceil(ctx/block_size) are never read
 *   context_lens [num_seqs]; 0 gives a zero output row
 *   out          [num_seqs][num_q_heads][d] in out_dtype, strides os_seq / os_head
 * kv head of query head h is h / (num_q_heads / num_kv_heads).
 * `num_blocks` is the number of physical blocks behind k/v_packed and k/v_norms: table
 * entries inside a context are clamped into [0, num_blocks), so a corrupt entry reads a wrong
 * block of the cache, never memory outside it.
 * `workspace` (device, >= akv_paged_attn_workspace_bytes(...), 256-byte aligned) holds the
 * rotated queries and the split partials; the caller allocates it once.  One workspace may
 * serve calls of any batch size up to the one it was sized for; calls that share a workspace
 * must not overlap in time.
 * ------------------------------------------------------------------------------- */
size_t akv_paged_attn_workspace_bytes(int num_seqs, int num_q_heads, int d);
int akv_paged_attn(const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head,
                   const uint8_t* k_packed, int64_t kps_blk, int64_t kps_pos, int64_t kps_head,
                   const float* k_norms, int64_t kns_blk, int64_t kns_pos, int64_t kns_head,
                   const uint8_t* v_packed, int64_t vps_blk, int64_t vps_pos, int64_t vps_head,
                   const float* v_norms, int64_t vns_blk, int64_t vns_pos, int64_t vns_head,
                   const void* block_tables, int bt_itype, int64_t bt_stride,
                   const void* context_lens, int cl_itype,
                   const void* rot_prep, const float* centroids, int bits,
                   void* out, int out_dtype, int64_t os_seq, int64_t os_head,
                   int num_seqs, int num_q_heads, int num_kv_heads, int d,
                   int block_size, int64_t num_blocks, int64_t max_blocks_per_seq, float scale,
                   void* workspace, size_t workspace_bytes, void* stream);

/* akv_paged_attn without a workspace argument.  No counterpart in the reference: it is for callers
 * that cannot allocate and cannot bring a workspace -- code under HIP-graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  The rotated queries, split partials and cached tables
 * live in one fixed array of akv_paged_attn_static_scratch_bytes() (32 MiB) inside the library's
 * device image, held by every GPU the library runs on until the process ends.  The call allocates
 * and frees nothing.  A batch whose akv_paged_attn_workspace_bytes(...) exceeds the array is
 * refused with AKV_ERR_WORKSPACE (at 32 query heads and head_dim 128: up to 64 sequences).  All
 * calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams,
 * two threads) race; calls on one stream, or otherwise ordered, are fine, whatever their sizes.
 * Results are those of akv_paged_attn bit for bit. */
size_t akv_paged_attn_static_scratch_bytes(void);
int akv_paged_attn_static(const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head,
                          const uint8_t* k_packed, int64_t kps_blk, int64_t kps_pos, int64_t kps_head,
                          const float* k_norms, int64_t kns_blk, int64_t kns_pos, int64_t kns_head,
                          const uint8_t* v_packed, int64_t vps_blk, int64_t vps_pos, int64_t vps_head,
                          const float* v_norms, int64_t vns_blk, int64_t vns_pos, int64_t vns_head,
                          const void* block_tables, int bt_itype, int64_t bt_stride,
                          const void* context_lens, int cl_itype,
                          const void* rot_prep, const float* centroids, int bits,
                          void* out, int out_dtype, int64_t os_seq, int64_t os_head,
                          int num_seqs, int num_q_heads, int num_kv_heads, int d,
                          int block_size, int64_t num_blocks, int64_t max_blocks_per_seq, float scale,
                          void* stream);

/* Status of the most recent akv_paged_attn / akv_hybrid_paged_attn call that used `workspace`
 * (no counterpart in the reference).  Inside the main kernel pairs of wavefronts hand chunks to
 * each other through counters with BOUNDED waits, so that a kernel always finishes; a wait
 * that gives up marks the call, whose outputs are then all NaN.  This waits for `stream` and
 * copies the mark to *flags (host pointer): 0 = clean, bit 0 = a hand-off wait gave up.
 * workspace == NULL asks about the most recent akv_paged_attn_static call on the current device
 * (0 when there has been none).
 * akv_debug_set_handoff_spin_limit changes the number of polls such a wait makes (negative =
 * the default, 65536); it exists so that a test can exercise the failure path from the host
 * (0 polls: every wait gives up at once, every kernel still runs to its end).  The akv_debug_* and
 * akv_profile_* switches are process-global words read at each launch and are not synchronised: set them
 * from one thread while no call of another thread is being issued. */
int akv_paged_attn_status(const void* workspace, int* flags, void* stream);
int akv_debug_set_handoff_spin_limit(int polls);

/* A kernel that only reads: `bytes` of device memory at `src` (16-byte aligned) are summed, one word per
 * workgroup goes to `sink256` (256 bytes of device memory).  For benchmarks: timed through akv_profile_* like
 * the dominant kernels, it says what a plain streaming read reaches on the device at hand, next to the 8 TB/s
 * the roofline figures are quoted against.  No counterpart in the reference. */
int akv_debug_read_probe(const void* src, size_t bytes, void* sink256, void* stream);

/* ---------------------------------------------------------------------------------
 * HybridTurboQuant, mode tq35 with calibrate_uniform() groups (dims 0..63 at 3-bit MSE,
 * dims 64..127 at 2-bit MSE, each with a 1-bit QJL residual sketch and fp16 norms inside
 * the 64-byte row) -- aither_kvcache/hybrid_quantizer.py:616-779 (encode), :785-933 (decode).
 * `hyb_table` is a device float32[AKV_HYB_TABLE_FLOATS] laid out as
 *   [0,64)    group-0 Hadamard signs   [64,128)  group-1 Hadamard signs
 *   [128,192) group-0 QJL signs        [192,256) group-1 QJL signs
 *   [256,264) group-0 centroids (8)    [264,268) group-1 centroids (4)
 *   [268,275) group-0 boundaries (7)   [275,278) group-1 boundaries (3)
 * head_dim is 128.
 * ------------------------------------------------------------------------------- */
#define AKV_HYB_TABLE_FLOATS 288
#define AKV_HYB_PACKED_BYTES 64
int akv_hybrid_encode(const void* x, int x_dtype, int64_t n, int64_t x_stride,
                      const float* hyb_table, uint8_t* out, int64_t out_stride_bytes, void* stream);
/* Paged form: the encode half of tq::hybrid_decode_step, aither_kvcache/vllm/hooks.py:271-284;
 * same skipping rule as akv_encode_paged. */
int akv_hybrid_encode_paged(const void* x, int x_dtype, int64_t num_tokens, int num_kv_heads,
                            int64_t xs_token, int64_t xs_head,
                            const void* slot_mapping, int slot_itype, const float* hyb_table,
                            uint8_t* out, int64_t ps_blk, int64_t ps_pos, int64_t ps_head,
                            int block_size, int64_t max_blocks, void* stream);
/* K and V of a step in one call (both tensors with the strides given, both caches with the strides given): the two
 * encodes of tq::hybrid_decode_step, aither_kvcache/vllm/hooks.py:271-284; one launch while the call is small. */
int akv_hybrid_encode_paged_kv(const void* x_k, const void* x_v, int x_dtype, int64_t num_tokens, int num_kv_heads,
                               int64_t xs_token, int64_t xs_head,
                               const void* slot_mapping, int slot_itype, const float* hyb_table,
                               uint8_t* out_k, uint8_t* out_v, int64_t ps_blk, int64_t ps_pos, int64_t ps_head,
                               int block_size, int64_t max_blocks, void* stream);
int akv_hybrid_decode(const uint8_t* packed, int64_t packed_stride_bytes, int64_t n,
                      const float* hyb_table, float* out, int64_t out_stride, void* stream);
/* Decode attention over a tq35 paged cache.  The reference has no fused kernel for this: its
 * tq::hybrid_decode_step (aither_kvcache/vllm/hooks.py:240-345) decompresses every addressed
 * block and runs dense attention; this computes the same softmax(q K^T * scale) V directly on
 * the packed rows (float32 accumulation).  `scale` is explicit, as at hooks.py:341.
 * num_blocks, workspace sharing and akv_paged_attn_status as for akv_paged_attn. */
size_t akv_hybrid_paged_attn_workspace_bytes(int num_seqs, int num_q_heads);
int akv_hybrid_paged_attn(const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head,
                          const uint8_t* k_cache, int64_t kps_blk, int64_t kps_pos, int64_t kps_head,
                          const uint8_t* v_cache, int64_t vps_blk, int64_t vps_pos, int64_t vps_head,
                          const void* block_tables, int bt_itype, int64_t bt_stride,
                          const void* context_lens, int cl_itype, const float* hyb_table,
                          void* out, int out_dtype, int64_t os_seq, int64_t os_head,
                          int num_seqs, int num_q_heads, int num_kv_heads,
                          int block_size, int64_t num_blocks, int64_t max_blocks_per_seq, float scale,
                          void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------
 * HybridTurboQuant, mode tq25 with calibrate_uniform() groups (dims 0..31 at 2-bit MSE, dims 32..127
 * at 1-bit MSE, each with a 1-bit QJL residual sketch and fp16 norms inside the 44-byte row; the 96
 * coordinates of group 1 are transformed as a 64-point and a 32-point block and divided by sqrt(96)) --
 * aither_kvcache/hybrid_quantizer.py:59-65 (mode), :154-193 (transform of 96 points), :616-779 (encode),
 * :785-933 (decode).  Same arguments as the tq35 entry points above; `hyb_table` is a device
 * float32[AKV_HYB_TABLE_FLOATS] laid out as
 *   [0,128)   Hadamard signs in coordinate order (group 0's 32, then group 1's 96)
 *   [128,256) QJL signs likewise
 *   [256,260) group-0 centroids (4)     [260,262) group-1 centroids (2)
 *   [262,265) group-0 boundaries (3)    [265]     group-1 boundary
 * Rows: [0,8) group-0 codes, [8,12) group-0 sign bits, [12,16) group-0 norm and residual norm (fp16 LE),
 * [16,28) group-1 codes, [28,40) group-1 sign bits, [40,44) group-1 norms.  head_dim is 128.
 * akv_hybrid25_paged_attn is the attention of tq::hybrid_decode_step (aither_kvcache/vllm/hooks.py:240-345)
 * on such rows; its workspace has the size akv_hybrid_paged_attn_workspace_bytes gives.
 * ------------------------------------------------------------------------------- */
#define AKV_HYB25_PACKED_BYTES 44
int akv_hybrid25_encode(const void* x, int x_dtype, int64_t n, int64_t x_stride,
                        const float* hyb_table, uint8_t* out, int64_t out_stride_bytes, void* stream);
int akv_hybrid25_encode_paged(const void* x, int x_dtype, int64_t num_tokens, int num_kv_heads,
                              int64_t xs_token, int64_t xs_head,
                              const void* slot_mapping, int slot_itype, const float* hyb_table,
                              uint8_t* out, int64_t ps_blk, int64_t ps_pos, int64_t ps_head,
                              int block_size, int64_t max_blocks, void* stream);
int akv_hybrid25_encode_paged_kv(const void* x_k, const void* x_v, int x_dtype, int64_t num_tokens, int num_kv_heads,
                                 int64_t xs_token, int64_t xs_head,
                                 const void* slot_mapping, int slot_itype, const float* hyb_table,
                                 uint8_t* out_k, uint8_t* out_v, int64_t ps_blk, int64_t ps_pos, int64_t ps_head,
                                 int block_size, int64_t max_blocks, void* stream);
int akv_hybrid25_decode(const uint8_t* packed, int64_t packed_stride_bytes, int64_t n,
                        const float* hyb_table, float* out, int64_t out_stride, void* stream);
int akv_hybrid25_paged_attn(const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head,
                            const uint8_t* k_cache, int64_t kps_blk, int64_t kps_pos, int64_t kps_head,
                            const uint8_t* v_cache, int64_t vps_blk, int64_t vps_pos, int64_t vps_head,
                            const void* block_tables, int bt_itype, int64_t bt_stride,
                            const void* context_lens, int cl_itype, const float* hyb_table,
                            void* out, int out_dtype, int64_t os_seq, int64_t os_head,
                            int num_seqs, int num_q_heads, int num_kv_heads,
                            int block_size, int64_t num_blocks, int64_t max_blocks_per_seq, float scale,
                            void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------
 * TriAttention.decode_step -- aither_kvcache/triattention/attention.py:186-280 with
 * TrigSeriesScorer.score (scorer.py:115-208):
 *   k/v_indices [B][S][KVH][F] uint8; k/v_coeffs by coeff_bits (scorer.py:84-113):
 *     4   [B][S][KVH][F] uint8, hi nibble = even component, value = (code / 7.5 - 1) * scale
 *     8   [B][S][KVH][2F] uint8, even then odd component of each pair, (code / 127.5 - 1) * scale
 *     16  [B][S][KVH][F][2] fp16, the components themselves; k/v_scales are not read (may be NULL)
 *   k/v_scales [B][S][KVH] fp16, all contiguous; theta [d/2] float32
 *   (spectral.py:34-51); query [B][QH][d] (contiguous); query_pos [B] or NULL (= S);
 *   key_positions [B][S] or NULL (= 0..S-1); out [B][QH][d] float32.
 *   pre_rope != 0: the trigonometric series over key position - query position (scorer.py:180-199);
 *   pre_rope == 0: keys were stored after RoPE, the score is the plain sparse dot product
 *   (scorer.py:200-202) and the positions are not used.
 * ------------------------------------------------------------------------------- */
size_t akv_tri_decode_workspace_bytes(int batch, int num_q_heads, int d);
int akv_tri_decode_step(const void* query, int q_dtype,
                        const uint8_t* k_indices, const void* k_coeffs, const void* k_scales,
                        const uint8_t* v_indices, const void* v_coeffs, const void* v_scales,
                        const float* theta,
                        const void* query_pos, int qp_itype,
                        const void* key_positions, int kp_itype,
                        float* out, int batch, int64_t seq_len, int num_q_heads, int num_kv_heads,
                        int d, int num_freqs, int coeff_bits, int pre_rope,
                        void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------
 * TrigSeriesScorer.score -- aither_kvcache/triattention/scorer.py:115-208: the pre-softmax logits alone,
 * for callers that add a mask (TriAttention.forward, attention.py:148-166) or inspect the scores.
 * Arguments as for akv_tri_decode_step; out [B][QH][S] float32, contiguous.
 * ------------------------------------------------------------------------------- */
int akv_tri_scores(const void* query, int q_dtype,
                   const uint8_t* k_indices, const void* k_coeffs, const void* k_scales,
                   const float* theta,
                   const void* query_pos, int qp_itype,
                   const void* key_positions, int kp_itype,
                   float* out, int batch, int64_t seq_len, int num_q_heads, int num_kv_heads,
                   int d, int num_freqs, int coeff_bits, int pre_rope, void* stream);

/* ---------------------------------------------------------------------------------
 * TriAttention.decode_step over a paged spectral cache: what the reference does per sequence
 * with SpectralKVCache.fetch_sequence (aither_kvcache/triattention/cache.py:163-198; block
 * layout :9-15) followed by decode_step, for a whole batch and without the gather.
 *   k/v_indices, k/v_coeffs [num_blocks][block_size][KVH][F] uint8, k/v_scales
 *   [num_blocks][block_size][KVH] fp16, contiguous; block_tables [B][>= ceil(ctx/block_size)]
 *   (row stride bt_stride elements; entries past the context are never dereferenced for
 *   ctx > 0); context_lens [B], clamped to max_blocks_per_seq * block_size; key positions are
 *   0..ctx-1; query_pos [B] or NULL (= ctx); out [B][QH][d] float32, zeros where ctx == 0.
 *   Coefficients are int4 (the only width the reference's cache stores, cache.py:66-85); pre_rope as for
 *   akv_tri_decode_step.
 * Workspace as for akv_tri_decode_step.  Built for d = 128, num_freqs = 12, at most 8 kv heads,
 * 4-byte aligned arrays, max_blocks_per_seq * block_size < 2^30 and num_blocks * block_size * KVH < 2^32
 * (blocks of 1 or 2 tokens: arrays below 4 GB); anything else returns AKV_ERR_UNSUPPORTED (gather, then
 * akv_tri_decode_step).  Blocks of 1 .. 64 tokens (a power of two) in arrays below 4 GB take the shortest
 * path: rows by 32-bit offsets and no division per chunk.
 * ------------------------------------------------------------------------------- */
int akv_tri_decode_paged(const void* query, int q_dtype,
                         const uint8_t* k_indices, const uint8_t* k_coeffs, const void* k_scales,
                         const uint8_t* v_indices, const uint8_t* v_coeffs, const void* v_scales,
                         const float* theta,
                         const void* query_pos, int qp_itype,
                         const void* block_tables, int bt_itype, int64_t bt_stride,
                         const void* context_lens, int cl_itype,
                         float* out, int batch, int64_t num_blocks, int block_size,
                         int64_t max_blocks_per_seq, int num_q_heads, int num_kv_heads,
                         int d, int num_freqs, int pre_rope,
                         void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------
 * SpectralKVEncoder.encode -- aither_kvcache/triattention/encoder.py:73-149
 * (the write side of TriAttention; TriAttention.encode_kv, attention.py:160-184, calls it for
 * keys and values): per vector the num_freqs RoPE pairs (dims 2i, 2i+1) of largest energy,
 * indices ascending; scale = max |kept coefficient| clamped at 1e-8; then by coeff_bits
 *   4   code = clamp(round((v / scale + 1) * 7.5), 0, 15); byte = code(even) << 4 | code(odd);
 *       coeffs [n][num_freqs] uint8                                                    (:118-133)
 *   8   code = clamp(round((v / scale + 1) * 127.5), 0, 255); coeffs [n][2 num_freqs] uint8, even then
 *       odd component of each pair                                                     (:135-147)
 *   16  coeffs [n][num_freqs][2] fp16 = the components rounded to fp16; scales = 1     (:107-115)
 *   x [n][d] (row stride x_stride elements); indices [n][num_freqs] uint8; scales [n] fp16.
 * Pairs of exactly equal energy are kept lowest index first (torch.topk leaves that open).
 * head_dim above 128 returns AKV_ERR_UNSUPPORTED.
 * ------------------------------------------------------------------------------- */
int akv_tri_encode(const void* x, int x_dtype, int64_t n, int d, int64_t x_stride, int num_freqs,
                   int coeff_bits, uint8_t* indices, void* coeffs, void* scales, void* stream);

/* Encode-on-write for the paged spectral cache: SpectralKVEncoder.encode (encoder.py:73-149, int4 coefficients)
 * of x [num_tokens][num_kv_heads][d] (element strides xs_token, xs_head) written straight into the block pool --
 * what the reference does token by token with SpectralKVCache.store_token (aither_kvcache/triattention/cache.py:
 * 106-140) after encoding.  slot_mapping [num_tokens]: slot = block * block_size + position; a token whose slot is
 * negative or not below num_slots (= num_blocks * block_size) is skipped.  indices, coeffs
 * [num_slots][num_kv_heads][num_freqs] uint8 and scales [num_slots][num_kv_heads] fp16, contiguous (the cache's
 * k_* or v_* tensors). */
int akv_tri_encode_paged(const void* x, int x_dtype, int64_t num_tokens, int num_kv_heads, int d,
                         int64_t xs_token, int64_t xs_head, int num_freqs,
                         const void* slot_mapping, int slot_itype, int64_t num_slots,
                         uint8_t* indices, uint8_t* coeffs, void* scales, void* stream);

/* ---------------------------------------------------------------------------------
 * Block selection for sparse decode attention -- aither_kvcache/block_selector.py.
 * The attention entry points take the filtered table and context lengths as they are.
 *
 * akv_block_rep_update: BlockSelector.update_reps (:282-292) = BlockRepresentativeCache.update
 *   (:66-101) + finalize of the touched blocks (:103-118).  For each of the n new tokens and each
 *   kv head, norm * centroids[high nibble] is added to acc_even[block][head][byte] and
 *   norm * centroids[low nibble] to acc_odd, the block's count goes up by one; then, unless
 *   rep_even/rep_odd are NULL, rep = acc / max(count, 1) for the blocks listed.  Block ids
 *   outside [0, max_blocks) are skipped.  4-bit codes.  counts is int32 (the reference keeps
 *   int16).  k_packed [n][kv_heads][packed_dim] with byte strides, k_norms [n][kv_heads] with
 *   element strides; acc_* / rep_* [max_blocks][kv_heads][packed_dim] float32, contiguous.
 * akv_block_rep_finalize: finalize (:103-118) for the blocks listed, or for all when
 *   block_indices is NULL.
 * akv_block_scores: score_blocks (:129-179).  q_even / q_odd [seqs][q_heads][half_d] float32
 *   (even / odd coordinates of the rotated query), scores [seqs][max_blocks_per_seq] float32;
 *   table columns at or beyond ceil(context / block_size) get -inf, table entries are clamped
 *   into [0, num_blocks).
 * akv_block_select: select_blocks (:182-236).  filtered_block_tables [seqs][max_selected] in the
 *   table's integer type: sink and recent columns, then the best-scoring ones, k =
 *   min(max_selected, max_blocks_per_seq) in all, in column order, zero padding behind;
 *   filtered_context_lens = min(context, k * block_size).  Equal scores: lower column first.
 * ------------------------------------------------------------------------------- */
int akv_block_rep_update(const void* block_indices, int idx_itype, int64_t n,
                         const uint8_t* k_packed, int64_t ps_tok, int64_t ps_head,
                         const float* k_norms, int64_t ns_tok, int64_t ns_head, const float* centroids,
                         float* acc_even, float* acc_odd, int32_t* counts, float* rep_even, float* rep_odd,
                         int64_t max_blocks, int num_kv_heads, int packed_dim, void* stream);
int akv_block_rep_finalize(const void* block_indices, int idx_itype, int64_t n,
                           const float* acc_even, const float* acc_odd, const int32_t* counts,
                           float* rep_even, float* rep_odd,
                           int64_t max_blocks, int num_kv_heads, int packed_dim, void* stream);
int akv_block_scores(const float* q_even, const float* q_odd, const float* rep_even, const float* rep_odd,
                     const void* block_tables, int bt_itype, int64_t bt_stride,
                     const void* context_lens, int cl_itype,
                     int num_seqs, int num_q_heads, int num_kv_heads, int half_d,
                     int64_t max_blocks_per_seq, int block_size, int64_t num_blocks,
                     float* scores, void* stream);
int akv_block_select(const float* scores, const void* block_tables, int bt_itype, int64_t bt_stride,
                     const void* context_lens, int cl_itype, int num_seqs, int64_t max_blocks_per_seq,
                     int block_size, int max_selected, int num_sink_blocks, int num_recent_blocks,
                     void* filtered_block_tables, void* filtered_context_lens, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AITHERKV_H */
