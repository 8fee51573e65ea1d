/*
 * kvx.h -- C ABI of libkvx: attention-with-score-sums and KV-cache kernels for AMD MI355X (gfx950).
 *
 * Everything here is plain C: raw device pointers, element strides, sizes and an opaque stream
 * handle (a hipStream_t passed as void*; NULL = the null stream). No entry point allocates or
 * frees memory, none synchronises the stream, none throws. Every call returns KVX_OK (0) or a
 * KVX_ERR_* code; kvx_last_error() then holds a message for the calling thread.
 *
 * Each entry point names the interface of awslabs/keys_values (the "reference", paths relative
 * to its repository root) that it stands in for.
 *
 * Conventions
 *   B      batch size                 Hq     query heads          Hkv   key/value heads
 *   G      Hq / Hkv (group size)      D      head size (64, 128 or 256)
 *   q_len  queries per call           kv_len cache slots visible to the call
 *   Tensors are addressed as base + b*stride_b + h*stride_h + t*stride_t + d with the head
 *   dimension contiguous; strides are in ELEMENTS of the tensor's own type. This covers both the
 *   reference's (B, H, T, D) cache views (keys_values/kvcache/buffers.py:538-541) and the
 *   (B, T, H, D) layout of its extension (keys_values/csrc/bindings.cpp:98-122) without a copy.
 *   token_positions is int32 (B, Hkv, kv_len) (keys_values/kvcache/attn_weights.py:466-470);
 *   a NULL pointer means arange(kv_len) (keys_values/attention/attention_utils.py:425-432).
 *   A query at chunk offset i may see slot k iff token_positions[b,h,k] <= input_pos + i
 *   (keys_values/attention/attention_utils.py:238-247).
 *   Score-sums W are fp32 (B, Hkv, kv_len): sum over queries, MEAN over the G grouped heads
 *   (keys_values/attention/base.py:707-725, keys_values/attention/flashinfer_wrapper.py:269-273).
 *   LSE is fp32 (B, q_len, Hq), base 2 (keys_values/csrc/kernels/sdpa_prefill.cu:509-512).
 */
#ifndef KVX_H
#define KVX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KVX_VERSION 103 /* major*10000 + minor*100 + patch */

enum kvx_status {
  KVX_OK = 0,
  KVX_ERR_INVALID = 1,     /* bad shape / stride / NULL pointer / range  (reference: TORCH_CHECK, bindings.cpp:37-62) */
  KVX_ERR_UNSUPPORTED = 2, /* head size or dtype outside what the kernels cover (reference: NotImplementedError,
                              flashinfer_wrapper.py:425-432) */
  KVX_ERR_HIP = 3,         /* a HIP runtime call failed (reference: TORCH_CHECK(err == cudaSuccess), bindings.cpp:486,955) */
  KVX_ERR_WORKSPACE = 4    /* workspace pointer NULL or smaller than kvx_*_workspace_bytes() */
};

/* Storage type of the K/V cache handed to the attention kernels. */
enum kvx_kv_dtype {
  KVX_KV_BF16 = 0, /* bfloat16 rows */
  KVX_KV_U8 = 1,   /* uint8 codes + per-row fp32 scale and int32 zero point (the reference's
                      "torch-quantized8" store, keys_values/kvcache/quantize/pytorch.py:281-295);
                      rows are dequantised inside the kernel exactly as
                      keys_values/kvcache/quantize/pytorch.py:143-154,467-478 would, i.e. to bf16 */
  KVX_KV_F16 = 3,  /* float16 rows; q and o are then float16 as well (the reference's extension takes float16 and
                      bfloat16, keys_values/csrc/bindings.cpp:207, keys_values/attention/flashinfer_wrapper.py:311-319).
                      KVX_KV_BF16, KVX_KV_U8 and KVX_KV_U4 go with bfloat16 q and o. */
  KVX_KV_U4 = 2,   /* the 4-bit store of the same quantiser ("torch-quantized4"): rows of D/2 bytes, byte j =
                      code[j] << 4 | code[j + D/2] (keys_values/kvcache/quantize/pytorch.py:384-393,457-465),
                      same per-row state; strides of k / v count bytes */
  KVX_KV_U8_F16 = 4, /* KVX_KV_U8 / KVX_KV_U4 for a float16 model: the rows were float16 when they were quantised, */
  KVX_KV_U4_F16 = 5  /* they dequantise to float16 (the quantiser casts back to its source type,
                        keys_values/kvcache/quantize/pytorch.py:333,478), and q and o are float16 */
};

/* One attention call. Unused pointers are NULL. All strides in elements. */
typedef struct kvx_sdpa_args {
  int32_t B, Hq, Hkv, q_len, kv_len, D;
  int32_t input_pos;   /* position of the first query; >= 0 */
  int32_t kv_dtype;    /* enum kvx_kv_dtype */
  float sm_scale;      /* softmax scale, e.g. 1/sqrt(D) */
  int32_t num_splits;  /* KV splits for prefill/decode; 0 = library heuristic */

  const void* q;       /* bf16 (fp16 with KVX_KV_F16) (B, Hq, q_len, D) by strides */
  int64_t q_stride_b, q_stride_h, q_stride_t;
  const void* k;       /* bf16, fp16 or uint8 (B, Hkv, kv_len, D) by strides */
  int64_t k_stride_b, k_stride_h, k_stride_t;
  const void* v;
  int64_t v_stride_b, v_stride_h, v_stride_t;
  /* KVX_KV_U8 only: per-row state (B, Hkv, kv_len), strides shared by the four arrays */
  const float* k_scale;
  const int32_t* k_zp;
  const float* v_scale;
  const int32_t* v_zp;
  int64_t qs_stride_b, qs_stride_h;

  const int32_t* token_positions; /* (B, Hkv, kv_len) or NULL */
  int64_t tp_stride_b, tp_stride_h;

  void* o;             /* bf16 (fp16 with KVX_KV_F16) (B, Hq, q_len, D) by strides */
  int64_t o_stride_b, o_stride_h, o_stride_t;
  float* lse;          /* fp32 (B, q_len, Hq) contiguous, base 2; output of prefill/decode, input of score_sum */
  float* w;            /* fp32 (B, Hkv, kv_len) contiguous score-sums, or NULL */

  void* workspace;     /* scratch, kvx_sdpa_*_workspace_bytes(); may be NULL when that returns 0 */
  size_t workspace_bytes;

  /* kvx_sdpa_decode / kvx_sdpa_decode_h2o with score-sums only, optional (NULL: not wanted): one device uint32 that the
   * call sets to the number of (batch, KV head, split) workgroups whose logits went through the fp32 scratch in HBM
   * instead of staying on the chip -- all of them when the splits are too long for the LDS or that form is switched
   * off, else those whose bounded wait for their row ran out (normally 0; such a call is about 15 % slower). */
  uint32_t* decode_scratch_splits;
} kvx_sdpa_args;

/* ---- library ------------------------------------------------------------------------------- */

/* Library version (KVX_VERSION of the build). */
int kvx_version(void);

/* Message of the last failing call on this thread ("" if none). The pointer stays valid until
 * the next failing call on the same thread. */
const char* kvx_last_error(void);

/* Replaces is_available() / get_device_count() of the reference extension module
 * (keys_values/csrc/bindings.cpp:1722-1735): number of visible HIP devices whose architecture is
 * gfx950, 0 if none (never fails). */
int kvx_device_count(void);

/* Replaces get_device_info(device_id) (keys_values/csrc/bindings.cpp:1733-1735). Writes a
 * NUL-terminated description ("name, arch, CUs, LDS per CU, memory") into buf. */
int kvx_device_info(int device, char* buf, size_t buf_len);

/* ---- attention ----------------------------------------------------------------------------- */

/* Chunked-prefill attention: O = softmax(s*Q K^T + mask) V and the base-2 log-sum-exp per query row.
 * Stands in for sdpa_prefill(..., return_lse=True) of the reference extension
 * (keys_values/csrc/bindings.cpp:511-958, keys_values/attention/flashinfer_ops.py:302-370) and for
 * the FlashInfer prefill kernel behind it (keys_values/csrc/kernels/sdpa_prefill.cu:34-181,
 * 1182-1256); unlike those it takes token_positions directly, so the caller does not reorder the
 * cache (keys_values/attention/sdpa_wrapper.py:352-369). args->lse may be NULL if not wanted;
 * args->w is ignored. */
int kvx_sdpa_prefill(const kvx_sdpa_args* args, void* stream);
size_t kvx_sdpa_prefill_workspace_bytes(const kvx_sdpa_args* args);

/* Per-key score-sums from Q, K and the log-sum-exp of a preceding kvx_sdpa_prefill:
 * W[b,h,k] = (1/G) * sum_{i,g} exp2(s*log2(e)*q_{i,g}.k - lse[b,i,h*G+g]) * [tp[b,h,k] <= input_pos+i].
 * Stands in for triton_score_sum / _score_sum_kernel
 * (keys_values/attention/flashinfer_wrapper.py:51-273). Deterministic: every W element is owned by
 * one wavefront, no atomics. Reads args->lse, writes args->w; o and v are ignored. args->workspace is optional:
 * given kvx_sdpa_prefill_workspace_bytes(args) bytes, a short cache (too few keys to give every compute unit a
 * workgroup) has its query rows split over more workgroups, whose partial sums are added in a fixed order. */
int kvx_score_sum(const kvx_sdpa_args* args, void* stream);

/* kvx_sdpa_prefill followed by kvx_score_sum on the same stream: the whole
 * FlashInferSDPA._flashinfer_sdpa_fused_prefill step
 * (keys_values/attention/flashinfer_wrapper.py:476-494). args->lse must be given (it carries the
 * log-sum-exp between the two kernels); workspace as for kvx_sdpa_prefill. */
int kvx_sdpa_prefill_weights(const kvx_sdpa_args* args, void* stream);

/* Single-token decode (q_len == 1): O over the whole cache and, if args->w is set, the score-sums
 * W = (1/G) sum_g softmax_g. No mask: the new token is the newest
 * (keys_values/attention/flashinfer_wrapper.py:471-481, keys_values/attention/flashinfer_ops.py:250-275).
 * Stands in for sdpa_decode of the reference extension (keys_values/csrc/bindings.cpp:86-489) and
 * optimized_batched_decode_kernel (keys_values/csrc/kernels/sdpa_decode.cu:616-898). One workgroup
 * per (batch, KV head, split) serves all G query heads, so K and V are read once. With args->w set, a
 * split keeps its logits on the chip, waits (boundedly) until the other splits of its (batch, KV head) row
 * have published their partial maxima and sums, and writes its part of W itself; the workspace holds
 * the split partials, the rows' arrival counters and room for the fp32 logits (B, Hq, kv_len) of the
 * splits that are too long for that or whose wait ran out. args->lse optional. */
int kvx_sdpa_decode(const kvx_sdpa_args* args, void* stream);
size_t kvx_sdpa_decode_workspace_bytes(const kvx_sdpa_args* args);

/* Single-token decode fused with the H2O bookkeeping that follows it in one cache step
 * (DefaultKVCache.forward for one new token: self.mha(...) then self._update(...),
 * keys_values/kvcache/base.py:583-595; H2OKVCache._compute_scores, keys_values/kvcache/h2o.py:175-196;
 * the argsort whose first entry the next step consumes, keys_values/kvcache/attn_weights.py:773-774):
 * kvx_sdpa_decode followed by kvx_h2o_update_select with k = 1, except that the score-sums go
 * straight from the kernel that produces them into scores += W and the per-row (value, slot)
 * minimum, without a round trip through memory. h->k must be 1, h->kv_len == args->kv_len;
 * h->w is ignored; args->w may be NULL (W is then not written out). h->workspace as for
 * kvx_h2o_update_select; args->workspace from kvx_sdpa_decode_h2o_workspace_bytes. */
struct kvx_h2o_args;
int kvx_sdpa_decode_h2o(const kvx_sdpa_args* args, const struct kvx_h2o_args* h, void* stream);
size_t kvx_sdpa_decode_h2o_workspace_bytes(const kvx_sdpa_args* args);

/* Process-wide switches of the decode kernels' weights route, for tests and measurement; no counterpart in the
 * reference. resident: 0 sends every split's logits through the workspace and the tail kernel, 1 keeps them on the
 * chip where they fit. spin_limit: polls a split spends waiting for the other splits of its row before it gives up
 * and takes the workspace route (0 = never wait; clamped to 2^20). poll_sleep: pause between two polls in units of
 * 512 cycles (clamped to 64). A negative value restores that switch to its default: the environment variables
 * KVX_DECODE_RESIDENT / KVX_DECODE_SPIN_LIMIT / KVX_DECODE_POLL_SLEEP as read once at the first decode call
 * (else 1, 32768, 4). A workspace size query and the call it is for must see the same setting of `resident`. */
void kvx_decode_tuning(int resident, int spin_limit, int poll_sleep);

/* ---- cache: quantiser ---------------------------------------------------------------------- */

/* Affine 8-bit row quantiser: for each row x[0..D) (bf16, upcast to fp32)
 *   scale = max((max - min) / 255, 1.1920929e-07);  zp = -(int32) rint(min / scale);
 *   code  = (uint8) clamp(rint(x * (1 / scale)) + zp, 0, 255)
 * bit-for-bit as TorchBasicQuantizer._quantize with MyPerChannelMinMaxObserver._calculate_qparams and
 * quantize_per_channel (keys_values/kvcache/quantize/pytorch.py:100-139,312-355).
 * x: bf16, `rows` rows of D elements, row r at x + r*x_row_stride. codes: uint8 rows*D contiguous.
 * scale / zp: one per row, contiguous. D in {64, 128, 256}. */
int kvx_quantize_rows(const void* x, int64_t x_row_stride, int64_t rows, int32_t D,
                      uint8_t* codes, float* scale, int32_t* zp, void* stream);

/* Inverse: out[r][d] = bf16( (float)((int32)code - zp) * scale ), as TorchBasicQuantizer._dequantize /
 * dequantize_per_channel (keys_values/kvcache/quantize/pytorch.py:143-154,411-478). */
int kvx_dequantize_rows(const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows,
                        int32_t D, void* out, int64_t out_row_stride, void* stream);

/* The 4-bit store of the same quantiser (num_bits = 4, keys_values/kvcache/quantize/pytorch.py:191-196):
 * scale = max((max - min) / 15, 1.1920929e-07), codes clamped to [0, 15], and two codes per byte,
 * byte j = code[j] << 4 | code[j + D/2] for j < D/2 (_compress_internal / _uncompress_internal,
 * keys_values/kvcache/quantize/pytorch.py:384-393,457-465). codes: rows * D/2 bytes, contiguous. */
int kvx_quantize_rows4(const void* x, int64_t x_row_stride, int64_t rows, int32_t D,
                       uint8_t* codes, float* scale, int32_t* zp, void* stream);
int kvx_dequantize_rows4(const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows,
                         int32_t D, void* out, int64_t out_row_stride, void* stream);

/* The four calls above with the number of bits (8 or 4) and the type of the rows as arguments: elem_dtype is
 * KVX_KV_BF16 or KVX_KV_F16. The quantiser upcasts any float type to fp32 and casts the dequantised values back to
 * the type it was built for (source_dtype, keys_values/kvcache/quantize/pytorch.py:333,478), so a float16 model's
 * store holds codes of float16 rows and dequantises to float16. */
int kvx_quantize_rows_typed(const void* x, int64_t x_row_stride, int64_t rows, int32_t D, int32_t bits, int32_t elem_dtype,
                            uint8_t* codes, float* scale, int32_t* zp, void* stream);
int kvx_dequantize_rows_typed(const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows, int32_t D,
                              int32_t bits, int32_t elem_dtype, void* out, int64_t out_row_stride, void* stream);

/* General form: a quantisation block is `nseg` segments of D contiguous bf16 values, segment s of block
 * (o, i) at x + o*x_stride_outer + i*x_stride_inner + s*x_stride_seg (strides in elements). With
 * nseg = n_query_groups and the segment stride that of the head axis this is blocks_over_heads=True
 * (one block per token over all heads, keys_values/kvcache/quantize/pytorch.py:235-245,333-336: the
 * values are transposed to (batch, slot, head, head_size) before they are flattened); nseg = 1 is the
 * row form above. bits is 8 or 4; with 4 bits byte j of a block holds code[j] << 4 | code[j + E/2],
 * E = nseg * D. Block (o, i) goes to codes + o*codes_stride_outer + i*E*bits/8 (bytes) and its state
 * to scale / zp [o*state_stride_outer + i]. E <= 8192, D a multiple of 16.
 * kvx_dequantize_blocks is the inverse with the same argument block (x is then the output). */
typedef struct kvx_block_quant_args {
  void* x; /* bf16; input of quantize, output of dequantize */
  int64_t x_stride_outer, x_stride_inner, x_stride_seg;
  int32_t n_outer, n_inner, nseg, D, bits;
  uint8_t* codes;
  int64_t codes_stride_outer; /* bytes */
  float* scale;
  int32_t* zp;
  int64_t state_stride_outer; /* elements */
  int32_t elem_dtype;         /* type of x: KVX_KV_BF16 (0) or KVX_KV_F16 */
} kvx_block_quant_args;
int kvx_quantize_blocks(const kvx_block_quant_args* args, void* stream);
int kvx_dequantize_blocks(const kvx_block_quant_args* args, void* stream);

/* ---- cache: write and H2O bookkeeping ------------------------------------------------------- */

/* Write `num` new tokens into the slots chosen by the previous selection, and do the bookkeeping
 * that AttnWeightsKVCache._forward_internal does around it
 * (keys_values/kvcache/attn_weights.py:510-635; update_token_positions :214-317;
 * DefaultKVCacheBuffers.set_slots, keys_values/kvcache/buffers.py:498-519;
 * _update_score_buffers_in_forward :636-681):
 *   slot = index[b,h,j];  token_pos[b,h,slot] = input_pos + j;  scores[b,h,slot] = 0;
 *   K[b,h,slot,:] = key[b,h,j,:];  V likewise.
 * With kv_dtype == KVX_KV_U8 the rows are quantised on the way in (same arithmetic as
 * kvx_quantize_rows) into codes + k_scale/k_zp/v_scale/v_zp.
 * index: int32 (B, Hkv, index_stride_h >= num) with index_stride_b / _h in elements.
 * key/value: bf16 (B, Hkv, num, D) by strides. scores may be NULL (no score buffer).
 *
 * Grace period (grace_num = num2 > 0; the cache is full and its last grace_period slots are a ring
 * of the most recent tokens, keys_values/kvcache/attn_weights.py:267-303,565-606). With
 * num1 = num - num2 and ring = grace_slots[j] (oldest ring slot first), job j does
 *   j <  num2: everything slot `ring` holds (K/V row, quantiser state, token position
 *              input_pos - grace_period + j, scores, v_norm, q_errors) moves to index[b,h,j];
 *              then the new token num1 + j goes into `ring` (position input_pos + num1 + j);
 *   j >= num2: the new token j - num2 goes into index[b,h,j] (position input_pos + j - num2).
 * A moved row of a quantised cache is dequantised and quantised again on its way to index[b,h,j], as
 * the reference's write does (the ring rows come out of its dequantised buffer,
 * keys_values/kvcache/quant_buffers.py:732-775); its q_errors entry moves unchanged. Slots in index
 * must lie outside the ring.
 *
 * replay_log (see the field comments) records the slots written.
 *
 * Further score buffers, same layout and strides as scores, NULL if the policy has none:
 *   v_norm   |value row|_2 in fp32 (VLengthInstantScoreMixin._initial_scores_in_forward,
 *            keys_values/kvcache/h2o.py:316-341);
 *   q_errors |k - dq(q(k))|_2 + |v - dq(q(v))|_2 of the new row, differences rounded to bf16 and
 *            norms in fp32 (QuantizedH2OKVCache._compute_quantization_errors,
 *            keys_values/kvcache/qh2o.py:130-176; keys_values/kvcache/quantize/pytorch.py:530-548).
 *            Needs KVX_KV_U8. */
typedef struct kvx_cache_write_args {
  int32_t B, Hkv, num, D, cache_len;
  int32_t input_pos;
  int32_t kv_dtype;
  const int32_t* index;
  int64_t index_stride_b, index_stride_h;
  const void* key;
  int64_t key_stride_b, key_stride_h, key_stride_t;
  const void* value;
  int64_t value_stride_b, value_stride_h, value_stride_t;
  void* k_cache; /* bf16 or uint8 (B, Hkv, cache_len, D) */
  int64_t kc_stride_b, kc_stride_h, kc_stride_t;
  void* v_cache;
  int64_t vc_stride_b, vc_stride_h, vc_stride_t;
  float* k_scale;
  int32_t* k_zp;
  float* v_scale;
  int32_t* v_zp;
  int64_t qs_stride_b, qs_stride_h;
  int32_t* token_pos; /* (B, Hkv, cache_len), or NULL: rows only (DefaultKVCacheBuffers.set_slots, no position bookkeeping) */
  int64_t tp_stride_b, tp_stride_h;
  float* scores; /* (B, Hkv, cache_len) or NULL */
  int64_t sc_stride_b, sc_stride_h;
  int32_t grace_num;          /* num2 <= min(num, grace_period); 0 = no ring move */
  int32_t grace_period;
  const int32_t* grace_slots; /* (grace_num) ring slots, shared by all (b, h) */
  float* v_norm;              /* (B, Hkv, cache_len) by sc_stride_*, or NULL */
  float* q_errors;            /* (B, Hkv, cache_len) by sc_stride_*, or NULL */
  /* Replay log (AttnWeightsReplayLog.append_position_index, keys_values/kvcache/attn_weights.py:125-151):
   * the slots index[b,h,j] this call writes to are recorded as uint32, entry p = log_pos + j of
   * (b, h) at replay_log[(p / log_blocksize) * log_stride_block + b * log_stride_b + h * log_stride_h
   * + p % log_blocksize]: blocks of log_blocksize positions, all blocks in one allocation.
   * log_pos = input_pos - cache_length of the first new token. NULL: nothing is recorded. */
  uint32_t* replay_log;
  int32_t log_blocksize;
  int64_t log_pos;
  int64_t log_stride_block, log_stride_b, log_stride_h;
} kvx_cache_write_args;
int kvx_cache_write(const kvx_cache_write_args* args, void* stream);

/* H2O score update and eviction choice, AttnWeightsKVCache._update with H2OKVCache._compute_scores
 * (keys_values/kvcache/attn_weights.py:721-783, keys_values/kvcache/h2o.py:146-199):
 *   scores[b,h,:kv_len] += w[b,h,:kv_len]           (skipped when w is NULL)
 *   next_index[b,h,0..k) = the k slots of scores[b,h,:limit] with the smallest value,
 *                          in ascending (value, slot) order, ties to the lower slot.
 * This is scores.argsort(-1)[..., :k]; the reference's topk(k, largest=False, sorted=False) returns
 * the same set in unspecified order. limit = cache_length - grace_period: the ring is never evicted.
 * With normalize != 0 the value compared is
 * scores / (input_pos - max(token_pos, prefill_len - 1)) (keys_values/kvcache/h2o.py:183-196);
 * token_pos then must be given. 1 <= k <= limit <= kv_len; up to 4096 slots are chosen per kernel launch,
 * a longer selection (up to the whole argsort, k = limit) takes ceil(k / 4096) launches and 8 bytes of
 * workspace per row.
 * scores rows at scores + b*sc_stride_b + h*sc_stride_h; w contiguous (B, Hkv, kv_len).
 * next_index: int32 (B, Hkv, k) contiguous.
 *
 * Policy variants (all pointers NULL / zero for plain H2O):
 *   v_norm   (same layout as scores): the amount added is (v_norm*w / sum_k(v_norm*w)) * q_len in
 *            place of w (VLengthInstantScoreMixin._instantaneous_score, keys_values/kvcache/h2o.py:297-314).
 *   q_errors (same layout as scores): the value compared becomes
 *            c*mm(value) + ((c-1)/2)*mm(q_errors) + (1-c), c = combination, where mm is the min-max
 *            normalisation over all (head, slot < limit) entries of one batch element
 *            (QuantizedH2OKVCache._modify_scores, keys_values/kvcache/qh2o.py:178-210).
 * With a variant the workspace also holds per-row statistics (kvx_h2o_workspace_bytes accounts for
 * them) and kvx_sdpa_decode_h2o is not available. */
typedef struct kvx_h2o_args {
  int32_t B, Hkv, kv_len, limit, k;
  int32_t normalize, input_pos, prefill_len;
  float* scores;
  int64_t sc_stride_b, sc_stride_h;
  const float* w;
  const int32_t* token_pos;
  int64_t tp_stride_b, tp_stride_h;
  int32_t* next_index;
  void* workspace;
  size_t workspace_bytes;
  const float* v_norm;   /* or NULL */
  const float* q_errors; /* or NULL */
  int32_t q_len;         /* queries behind w (v_norm only) */
  double combination;    /* c in [0, 1] (q_errors only); a double, as the reference's Python float */
} kvx_h2o_args;
int kvx_h2o_update_select(const kvx_h2o_args* args, void* stream);
size_t kvx_h2o_workspace_bytes(const kvx_h2o_args* args);

/* kvx_h2o_update_select for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. Same
 * arguments, same kernels, same results; args->workspace and args->workspace_bytes are ignored: the
 * scratch (the per-row minimum keys of k == 1, the per-row statistics of the q_errors combination)
 * lives in a device array of KVX_H2O_STATIC_SCRATCH_BYTES that is part of the library image, one copy
 * per GPU, held until the process ends. Calls whose kvx_h2o_workspace_bytes() exceeds that size return
 * KVX_ERR_WORKSPACE. The call allocates nothing and frees nothing; the first call on a device looks
 * the array's device address up (do that call outside a graph capture). All calls on one GPU share
 * the array: two calls that overlap on one GPU (different streams, no ordering between them) race;
 * calls on one stream, or ordered by events, do not. What the kernels need cleared they clear
 * themselves with a fill kernel, so the array's previous contents never matter. */
#define KVX_H2O_STATIC_SCRATCH_BYTES (128 * 1024)
int kvx_h2o_update_select_static(const kvx_h2o_args* args, void* stream);

/* ---- callers of the path: normalisation and rotary encoding of the new tokens ---------------- */

/* RMS normalisation of `rows` rows of `dim` bf16 values: out = (x / (|x|_2 / sqrt(dim) + eps)) * weight,
 * computed in fp32 with eps added to the norm, as RMSNorm.forward (keys_values/model.py:870-878).
 * weight: fp32 (dim). dim a multiple of 8, at most 8192. In place is allowed (out == x). */
int kvx_rmsnorm_rows(const void* x, int64_t x_row_stride, void* out, int64_t out_row_stride,
                     const float* weight, int64_t rows, int32_t dim, float eps, void* stream);

/* Residual add fused with the normalisation that follows it in a block (Block.forward,
 * keys_values/model.py:560-584: x = attention_output + x; ... norm_2(x)):
 *   x_out = bf16(x + delta);  out = RMSNorm(x_out) as kvx_rmsnorm_rows.
 * The sum is rounded to bf16 before it is normalised, as the two separate steps round. x_out may be x. */
int kvx_add_rmsnorm_rows(const void* x, int64_t x_row_stride, const void* delta, int64_t delta_row_stride,
                         void* x_out, int64_t x_out_row_stride, void* out, int64_t out_row_stride,
                         const float* weight, int64_t rows, int32_t dim, float eps, void* stream);

/* Gated activation of the MLP (LLaMAMLP.forward of litgpt, which keys_values/model.py builds on:
 * proj(silu(fc_1(x)) * fc_2(x))) on the output of ONE GEMM over the stacked fc_1 / fc_2 weights:
 *   out[r, j] = bf16( bf16(silu(gate_up[r, j])) * gate_up[r, dim + j] ),  silu(t) = t / (1 + exp(-t)) in fp32.
 * gate_up: bf16 (rows, 2 * dim) by row stride; out: bf16 (rows, dim). dim a multiple of 8. */
int kvx_swiglu_rows(const void* gate_up, int64_t gate_up_row_stride, void* out, int64_t out_row_stride,
                    int64_t rows, int32_t dim, void* stream);

/* Per-head normalisation of the new queries and keys followed by the rotary position encoding, in
 * place on the output of the QKV projection: what CausalSelfAttention.forward does between the
 * projection and the cache (keys_values/model.py:733-775: norm_q / norm_k, then
 * mha.pos_encoding -> apply_rope, keys_values/pos_encoding.py:34-44,201-238).
 * qkv: bf16 (B, num, (Hq + 2 Hkv) * D) by strides (elements), a token's heads stored as
 *      Hq query heads, Hkv key heads, Hkv value heads; the value heads are not touched.
 * q_weight / k_weight: fp32 (D) norm weights, or both NULL for no normalisation.
 * cos / sin: fp32 tables (table_rows, D / 2), row p = cos / sin of p * theta_j (half-split
 *      convention: element d is paired with d +- D/2). Token t of the chunk sits at input_pos + t.
 * D in {64, 128, 256}. */
int kvx_qk_norm_rope(void* qkv, int64_t stride_b, int64_t stride_t, int32_t B, int32_t num, int32_t Hq,
                     int32_t Hkv, int32_t D, const float* q_weight, const float* k_weight, float eps,
                     const float* cos, const float* sin, int32_t table_rows, int32_t input_pos,
                     void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KVX_H */
