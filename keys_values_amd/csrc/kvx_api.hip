// C ABI of libkvx: argument validation, error reporting and dispatch to the kernel launchers.
// The checks mirror what the reference extension enforces before launching
// (keys_values/csrc/bindings.cpp:37-62,98-178) and what keys_values/attention/sdpa_wrapper.py:24-47
// requires of the shapes; they also make sure no kernel can be launched on operands whose shape
// does not fit its indexing.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "kvx_common.h"

namespace kvx {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int hip_error(hipError_t e, const char* what) {
  return set_error(KVX_ERR_HIP, "HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
}

int num_cus() {
  static thread_local int cached_dev = -1;
  static thread_local int cached = 256;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return cached;
  if (dev != cached_dev) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cached = n;
    cached_dev = dev;
  }
  return cached;
}

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
bool mult8(int64_t x) { return (x & 7) == 0; }

int check_sdpa_common(const kvx_sdpa_args* a, const char* who, bool need_v_o) {
  KVX_REQUIRE(a != nullptr, KVX_ERR_INVALID, "%s: args is NULL", who);
  KVX_REQUIRE(a->B > 0 && a->Hq > 0 && a->Hkv > 0 && a->q_len > 0 && a->kv_len > 0, KVX_ERR_INVALID,
              "%s: sizes must be positive (B=%d Hq=%d Hkv=%d q_len=%d kv_len=%d)", who, a->B, a->Hq, a->Hkv, a->q_len,
              a->kv_len);
  KVX_REQUIRE(a->Hq % a->Hkv == 0, KVX_ERR_INVALID, "%s: Hq=%d must be a multiple of Hkv=%d", who, a->Hq, a->Hkv);
  // batch and head indices are grid dimensions, and B * Hq rows are counted in 32 bits
  KVX_REQUIRE(a->B <= 65535 && a->Hq <= 65535 && (int64_t)a->B * a->Hq < ((int64_t)1 << 24), KVX_ERR_UNSUPPORTED,
              "%s: B=%d, Hq=%d beyond 65535 each or 2^24 together", who, a->B, a->Hq);
  KVX_REQUIRE(kv_valid(a->kv_dtype), KVX_ERR_UNSUPPORTED, "%s: unknown kv_dtype %d", who, a->kv_dtype);
  KVX_REQUIRE(a->D == 64 || a->D == 128 || a->D == 256, KVX_ERR_UNSUPPORTED, "%s: head size %d not in {64, 128, 256}", who, a->D);
  const int row_elems = kv_is_u4(a->kv_dtype) ? a->D / 2 : a->D;  // elements of the cache's own type per row
  KVX_REQUIRE(a->input_pos >= 0, KVX_ERR_INVALID, "%s: input_pos=%d must be >= 0", who, a->input_pos);
  KVX_REQUIRE(a->sm_scale > 0.0f, KVX_ERR_INVALID, "%s: sm_scale must be positive", who);
  KVX_REQUIRE((int64_t)a->input_pos + a->q_len < INT32_MAX, KVX_ERR_INVALID, "%s: positions overflow int32", who);
  KVX_REQUIRE(a->q && a->k, KVX_ERR_INVALID, "%s: q and k must be given", who);
  KVX_REQUIRE(aligned16(a->q) && mult8(a->q_stride_b) && mult8(a->q_stride_h) && mult8(a->q_stride_t), KVX_ERR_INVALID,
              "%s: q must be 16-byte aligned with strides that are multiples of 8 elements", who);
  KVX_REQUIRE(aligned16(a->k) && mult8(a->k_stride_b) && mult8(a->k_stride_h) && mult8(a->k_stride_t), KVX_ERR_INVALID,
              "%s: k must be 16-byte aligned with strides that are multiples of 8 elements", who);
  KVX_REQUIRE(a->k_stride_t >= row_elems && a->q_stride_t >= 0, KVX_ERR_INVALID, "%s: bad k/q slot stride", who);
  if (need_v_o) {
    KVX_REQUIRE(a->v && a->o, KVX_ERR_INVALID, "%s: v and o must be given", who);
    KVX_REQUIRE(aligned16(a->v) && mult8(a->v_stride_b) && mult8(a->v_stride_h) && mult8(a->v_stride_t), KVX_ERR_INVALID,
                "%s: v must be 16-byte aligned with strides that are multiples of 8 elements", who);
    KVX_REQUIRE(aligned16(a->o) && mult8(a->o_stride_b) && mult8(a->o_stride_h) && mult8(a->o_stride_t), KVX_ERR_INVALID,
                "%s: o must be 16-byte aligned with strides that are multiples of 8 elements", who);
    KVX_REQUIRE(a->v_stride_t >= row_elems, KVX_ERR_INVALID, "%s: bad v slot stride", who);
  }
  if (!kv_is_plain(a->kv_dtype)) {
    KVX_REQUIRE(a->k_scale && a->k_zp, KVX_ERR_INVALID, "%s: quantised cache needs k_scale and k_zp", who);
    if (need_v_o) KVX_REQUIRE(a->v_scale && a->v_zp, KVX_ERR_INVALID, "%s: quantised cache needs v_scale and v_zp", who);
  }
  KVX_REQUIRE(a->num_splits >= 0, KVX_ERR_INVALID, "%s: num_splits must be >= 0", who);
  // the tiled kernels address a tile's rows with 32-bit byte offsets from the tile's base: 64 rows of the slot stride
  constexpr int64_t kMaxSlotStride = (int64_t)1 << 25;
  KVX_REQUIRE(a->k_stride_t <= kMaxSlotStride && (!need_v_o || a->v_stride_t <= kMaxSlotStride), KVX_ERR_UNSUPPORTED,
              "%s: slot strides above 2^25 elements are not supported", who);
  return KVX_OK;
}

}  // namespace
}  // namespace kvx

using namespace kvx;

extern "C" {

int kvx_version(void) { return KVX_VERSION; }

const char* kvx_last_error(void) { return g_err; }

int kvx_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  int good = 0;
  for (int i = 0; i < n; ++i) {
    hipDeviceProp_t pr;
    if (hipGetDeviceProperties(&pr, i) == hipSuccess && strncmp(pr.gcnArchName, "gfx950", 6) == 0) ++good;
  }
  return good;
}

int kvx_device_info(int device, char* buf, size_t buf_len) {
  KVX_REQUIRE(buf && buf_len > 0, KVX_ERR_INVALID, "kvx_device_info: empty buffer");
  hipDeviceProp_t pr;
  KVX_HIP(hipGetDeviceProperties(&pr, device));
  snprintf(buf, buf_len, "%s, %s, %d CUs, %zu KiB LDS per workgroup, %.1f GiB", pr.name, pr.gcnArchName,
           pr.multiProcessorCount, pr.sharedMemPerBlock / 1024, (double)pr.totalGlobalMem / (1024.0 * 1024.0 * 1024.0));
  return KVX_OK;
}

size_t kvx_sdpa_prefill_workspace_bytes(const kvx_sdpa_args* a) {
  if (check_sdpa_common(a, "kvx_sdpa_prefill_workspace_bytes", false) != KVX_OK) return 0;
  return sdpa_prefill_workspace(*a);
}

int kvx_sdpa_prefill(const kvx_sdpa_args* a, void* stream) {
  int rc = check_sdpa_common(a, "kvx_sdpa_prefill", true);
  if (rc != KVX_OK) return rc;
  KVX_REQUIRE(a->q_len <= a->kv_len, KVX_ERR_INVALID, "kvx_sdpa_prefill: q_len=%d exceeds kv_len=%d", a->q_len, a->kv_len);
  KVX_REQUIRE(aligned16(a->workspace), KVX_ERR_WORKSPACE, "kvx_sdpa_prefill: workspace must be 16-byte aligned");
  return launch_sdpa_prefill(*a, (hipStream_t)stream);
}

int kvx_score_sum(const kvx_sdpa_args* a, void* stream) {
  int rc = check_sdpa_common(a, "kvx_score_sum", false);
  if (rc != KVX_OK) return rc;
  KVX_REQUIRE(a->lse && a->w, KVX_ERR_INVALID, "kvx_score_sum: lse and w must be given");
  return launch_score_sum(*a, (hipStream_t)stream);
}

int kvx_sdpa_prefill_weights(const kvx_sdpa_args* a, void* stream) {
  int rc = check_sdpa_common(a, "kvx_sdpa_prefill_weights", true);
  if (rc != KVX_OK) return rc;
  KVX_REQUIRE(a->q_len <= a->kv_len, KVX_ERR_INVALID, "kvx_sdpa_prefill_weights: q_len=%d exceeds kv_len=%d", a->q_len,
              a->kv_len);
  KVX_REQUIRE(a->lse && a->w, KVX_ERR_INVALID, "kvx_sdpa_prefill_weights: lse and w must be given");
  KVX_REQUIRE(aligned16(a->workspace), KVX_ERR_WORKSPACE, "kvx_sdpa_prefill_weights: workspace must be 16-byte aligned");
  rc = launch_sdpa_prefill(*a, (hipStream_t)stream);
  if (rc != KVX_OK) return rc;
  return launch_score_sum(*a, (hipStream_t)stream);
}

size_t kvx_sdpa_decode_workspace_bytes(const kvx_sdpa_args* a) {
  if (check_sdpa_common(a, "kvx_sdpa_decode_workspace_bytes", false) != KVX_OK) return 0;
  return sdpa_decode_workspace(*a, false);
}

size_t kvx_sdpa_decode_h2o_workspace_bytes(const kvx_sdpa_args* a) {
  if (check_sdpa_common(a, "kvx_sdpa_decode_h2o_workspace_bytes", false) != KVX_OK) return 0;
  return sdpa_decode_workspace(*a, true);
}

void kvx_decode_tuning(int resident, int spin_limit, int poll_sleep) { set_decode_tuning(resident, spin_limit, poll_sleep); }

int kvx_sdpa_decode(const kvx_sdpa_args* a, void* stream) {
  int rc = check_sdpa_common(a, "kvx_sdpa_decode", true);
  if (rc != KVX_OK) return rc;
  KVX_REQUIRE(a->q_len == 1, KVX_ERR_INVALID, "kvx_sdpa_decode: q_len must be 1, got %d", a->q_len);
  const int G = a->Hq / a->Hkv;
  KVX_REQUIRE(G >= 1 && G <= 16 && (G <= 8 || a->D <= 128), KVX_ERR_UNSUPPORTED, "kvx_sdpa_decode: group size %d not in 1 .. 16 (1 .. 8 with head size 256)", G);
  KVX_REQUIRE(aligned16(a->workspace), KVX_ERR_WORKSPACE, "kvx_sdpa_decode: workspace must be 16-byte aligned");
  return launch_sdpa_decode(*a, nullptr, (hipStream_t)stream);
}

static int quantize_rows_checked(const char* who, const void* x, int64_t x_row_stride, int64_t rows, int32_t D, int32_t bits, int32_t elem_dtype,
                                 uint8_t* codes, float* scale, int32_t* zp, void* stream) {
  KVX_REQUIRE(D == 64 || D == 128 || D == 256, KVX_ERR_UNSUPPORTED, "%s: row length %d not in {64, 128, 256}", who, D);
  KVX_REQUIRE(bits == 8 || bits == 4, KVX_ERR_UNSUPPORTED, "%s: bits = %d, must be 4 or 8", who, bits);
  KVX_REQUIRE(elem_dtype == KVX_KV_BF16 || elem_dtype == KVX_KV_F16, KVX_ERR_UNSUPPORTED, "%s: elem_dtype %d is neither KVX_KV_BF16 nor KVX_KV_F16", who, elem_dtype);
  KVX_REQUIRE(rows >= 0, KVX_ERR_INVALID, "%s: rows must be >= 0", who);
  if (rows == 0) return KVX_OK;
  KVX_REQUIRE(x && codes && scale && zp, KVX_ERR_INVALID, "%s: NULL pointer", who);
  KVX_REQUIRE(aligned16(x) && mult8(x_row_stride) && x_row_stride >= D, KVX_ERR_INVALID,
              "%s: x must be 16-byte aligned, row stride a multiple of 8 and >= D", who);
  KVX_REQUIRE((reinterpret_cast<uintptr_t>(codes) & 7) == 0, KVX_ERR_INVALID, "%s: codes must be 8-byte aligned", who);
  return launch_quantize_rows(x, x_row_stride, rows, D, bits, elem_dtype == KVX_KV_F16, codes, scale, zp, (hipStream_t)stream);
}

static int dequantize_rows_checked(const char* who, const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows, int32_t D, int32_t bits,
                                   int32_t elem_dtype, void* out, int64_t out_row_stride, void* stream) {
  KVX_REQUIRE(D == 64 || D == 128 || D == 256, KVX_ERR_UNSUPPORTED, "%s: row length %d not in {64, 128, 256}", who, D);
  KVX_REQUIRE(bits == 8 || bits == 4, KVX_ERR_UNSUPPORTED, "%s: bits = %d, must be 4 or 8", who, bits);
  KVX_REQUIRE(elem_dtype == KVX_KV_BF16 || elem_dtype == KVX_KV_F16, KVX_ERR_UNSUPPORTED, "%s: elem_dtype %d is neither KVX_KV_BF16 nor KVX_KV_F16", who, elem_dtype);
  KVX_REQUIRE(rows >= 0, KVX_ERR_INVALID, "%s: rows must be >= 0", who);
  if (rows == 0) return KVX_OK;
  KVX_REQUIRE(codes && scale && zp && out, KVX_ERR_INVALID, "%s: NULL pointer", who);
  KVX_REQUIRE(aligned16(out) && mult8(out_row_stride) && out_row_stride >= D, KVX_ERR_INVALID,
              "%s: out must be 16-byte aligned, row stride a multiple of 8 and >= D", who);
  KVX_REQUIRE((reinterpret_cast<uintptr_t>(codes) & 7) == 0, KVX_ERR_INVALID, "%s: codes must be 8-byte aligned", who);
  return launch_dequantize_rows(codes, scale, zp, rows, D, bits, elem_dtype == KVX_KV_F16, out, out_row_stride, (hipStream_t)stream);
}

int kvx_quantize_rows(const void* x, int64_t x_row_stride, int64_t rows, int32_t D, uint8_t* codes, float* scale, int32_t* zp, void* stream) {
  return quantize_rows_checked("kvx_quantize_rows", x, x_row_stride, rows, D, 8, KVX_KV_BF16, codes, scale, zp, stream);
}
int kvx_dequantize_rows(const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows, int32_t D, void* out, int64_t out_row_stride,
                        void* stream) {
  return dequantize_rows_checked("kvx_dequantize_rows", codes, scale, zp, rows, D, 8, KVX_KV_BF16, out, out_row_stride, stream);
}
int kvx_quantize_rows4(const void* x, int64_t x_row_stride, int64_t rows, int32_t D, uint8_t* codes, float* scale, int32_t* zp, void* stream) {
  return quantize_rows_checked("kvx_quantize_rows4", x, x_row_stride, rows, D, 4, KVX_KV_BF16, codes, scale, zp, stream);
}
int kvx_dequantize_rows4(const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows, int32_t D, void* out, int64_t out_row_stride,
                         void* stream) {
  return dequantize_rows_checked("kvx_dequantize_rows4", codes, scale, zp, rows, D, 4, KVX_KV_BF16, out, out_row_stride, stream);
}
int kvx_quantize_rows_typed(const void* x, int64_t x_row_stride, int64_t rows, int32_t D, int32_t bits, int32_t elem_dtype, uint8_t* codes,
                            float* scale, int32_t* zp, void* stream) {
  return quantize_rows_checked("kvx_quantize_rows_typed", x, x_row_stride, rows, D, bits, elem_dtype, codes, scale, zp, stream);
}
int kvx_dequantize_rows_typed(const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows, int32_t D, int32_t bits,
                              int32_t elem_dtype, void* out, int64_t out_row_stride, void* stream) {
  return dequantize_rows_checked("kvx_dequantize_rows_typed", codes, scale, zp, rows, D, bits, elem_dtype, out, out_row_stride, stream);
}

static int check_blocks(const kvx_block_quant_args* a, const char* who) {
  KVX_REQUIRE(a != nullptr, KVX_ERR_INVALID, "%s: args is NULL", who);
  KVX_REQUIRE(a->n_outer >= 0 && a->n_inner >= 0 && a->nseg > 0 && a->D > 0, KVX_ERR_INVALID, "%s: bad sizes", who);
  KVX_REQUIRE(a->bits == 8 || a->bits == 4, KVX_ERR_UNSUPPORTED, "%s: bits = %d, must be 4 or 8", who, a->bits);
  KVX_REQUIRE(a->elem_dtype == KVX_KV_BF16 || a->elem_dtype == KVX_KV_F16, KVX_ERR_UNSUPPORTED, "%s: elem_dtype %d is neither KVX_KV_BF16 nor KVX_KV_F16",
              who, a->elem_dtype);
  KVX_REQUIRE(a->D % 16 == 0 && (int64_t)a->nseg * a->D <= 8192, KVX_ERR_UNSUPPORTED,
              "%s: D = %d must be a multiple of 16 and the block (nseg * D = %lld) at most 8192 values", who, a->D,
              (long long)a->nseg * a->D);
  if (a->n_outer == 0 || a->n_inner == 0) return KVX_OK;
  KVX_REQUIRE(a->x && a->codes && a->scale && a->zp, KVX_ERR_INVALID, "%s: NULL pointer", who);
  KVX_REQUIRE(aligned16(a->x) && mult8(a->x_stride_outer) && mult8(a->x_stride_inner) && mult8(a->x_stride_seg), KVX_ERR_INVALID,
              "%s: x must be 16-byte aligned with strides that are multiples of 8", who);
  KVX_REQUIRE((reinterpret_cast<uintptr_t>(a->codes) & 7) == 0 && (a->codes_stride_outer & 7) == 0, KVX_ERR_INVALID,
              "%s: codes must be 8-byte aligned", who);
  return KVX_OK;
}

int kvx_quantize_blocks(const kvx_block_quant_args* a, void* stream) {
  int rc = check_blocks(a, "kvx_quantize_blocks");
  if (rc != KVX_OK) return rc;
  return launch_quantize_blocks(*a, (hipStream_t)stream);
}

int kvx_dequantize_blocks(const kvx_block_quant_args* a, void* stream) {
  int rc = check_blocks(a, "kvx_dequantize_blocks");
  if (rc != KVX_OK) return rc;
  return launch_dequantize_blocks(*a, (hipStream_t)stream);
}

int kvx_cache_write(const kvx_cache_write_args* a, void* stream) {
  KVX_REQUIRE(a != nullptr, KVX_ERR_INVALID, "kvx_cache_write: args is NULL");
  KVX_REQUIRE(a->B > 0 && a->Hkv > 0 && a->num > 0 && a->cache_len > 0, KVX_ERR_INVALID, "kvx_cache_write: sizes must be positive");
  KVX_REQUIRE(kv_valid(a->kv_dtype), KVX_ERR_UNSUPPORTED, "kvx_cache_write: unknown kv_dtype %d", a->kv_dtype);
  KVX_REQUIRE(a->D == 64 || a->D == 128 || a->D == 256, KVX_ERR_UNSUPPORTED, "kvx_cache_write: head size %d not in {64, 128, 256}", a->D);
  KVX_REQUIRE(a->num <= a->cache_len, KVX_ERR_INVALID, "kvx_cache_write: num=%d exceeds cache_len=%d", a->num, a->cache_len);
  KVX_REQUIRE(a->index && a->key && a->value && a->k_cache && a->v_cache, KVX_ERR_INVALID, "kvx_cache_write: NULL pointer");
  KVX_REQUIRE(a->token_pos || a->grace_num == 0, KVX_ERR_INVALID, "kvx_cache_write: the ring move needs token_pos");
  KVX_REQUIRE(aligned16(a->key) && aligned16(a->value) && mult8(a->key_stride_b) && mult8(a->key_stride_h) &&
                  mult8(a->key_stride_t) && mult8(a->value_stride_b) && mult8(a->value_stride_h) && mult8(a->value_stride_t),
              KVX_ERR_INVALID, "kvx_cache_write: key/value must be 16-byte aligned with strides that are multiples of 8");
  KVX_REQUIRE(aligned16(a->k_cache) && aligned16(a->v_cache) && mult8(a->kc_stride_b) && mult8(a->kc_stride_h) &&
                  mult8(a->kc_stride_t) && mult8(a->vc_stride_b) && mult8(a->vc_stride_h) && mult8(a->vc_stride_t),
              KVX_ERR_INVALID, "kvx_cache_write: caches must be 16-byte aligned with strides that are multiples of 8");
  if (!kv_is_plain(a->kv_dtype))
    KVX_REQUIRE(a->k_scale && a->k_zp && a->v_scale && a->v_zp, KVX_ERR_INVALID, "kvx_cache_write: quantised cache needs scale / zero-point arrays");
  KVX_REQUIRE((int64_t)a->input_pos + a->num < INT32_MAX && a->input_pos >= 0, KVX_ERR_INVALID, "kvx_cache_write: bad input_pos");
  KVX_REQUIRE(a->grace_num >= 0 && a->grace_num <= a->num, KVX_ERR_INVALID, "kvx_cache_write: grace_num=%d must be in [0, num=%d]", a->grace_num, a->num);
  if (a->grace_num > 0) {
    KVX_REQUIRE(a->grace_slots, KVX_ERR_INVALID, "kvx_cache_write: grace_num > 0 needs grace_slots");
    KVX_REQUIRE(a->grace_num <= a->grace_period && a->grace_period < a->cache_len && a->input_pos >= a->grace_period, KVX_ERR_INVALID,
                "kvx_cache_write: need grace_num=%d <= grace_period=%d < cache_len=%d and input_pos=%d >= grace_period", a->grace_num,
                a->grace_period, a->cache_len, a->input_pos);
  }
  KVX_REQUIRE(!a->replay_log || (a->log_blocksize > 0 && a->log_pos >= 0), KVX_ERR_INVALID,
              "kvx_cache_write: replay log needs log_blocksize > 0 and log_pos >= 0");
  KVX_REQUIRE(!a->q_errors || !kv_is_plain(a->kv_dtype), KVX_ERR_INVALID, "kvx_cache_write: q_errors needs a quantised cache");
  return launch_cache_write(*a, (hipStream_t)stream);
}

size_t kvx_h2o_workspace_bytes(const kvx_h2o_args* a) { return a ? h2o_workspace(*a) : 0; }

static int check_h2o(const kvx_h2o_args* a, const char* who) {
  KVX_REQUIRE(a != nullptr, KVX_ERR_INVALID, "%s: h2o args is NULL", who);
  KVX_REQUIRE(a->B > 0 && a->Hkv > 0 && a->kv_len > 0, KVX_ERR_INVALID, "%s: sizes must be positive", who);
  KVX_REQUIRE(a->limit > 0 && a->limit <= a->kv_len, KVX_ERR_INVALID, "%s: limit=%d must be in [1, kv_len=%d]", who, a->limit, a->kv_len);
  KVX_REQUIRE(a->k >= 1 && a->k <= a->limit, KVX_ERR_INVALID, "%s: k=%d must be in [1, limit=%d]", who, a->k, a->limit);
  KVX_REQUIRE(a->scores && a->next_index, KVX_ERR_INVALID, "%s: NULL pointer", who);
  KVX_REQUIRE(!a->normalize || a->token_pos, KVX_ERR_INVALID, "%s: normalize needs token_pos", who);
  KVX_REQUIRE(!(a->v_norm && a->w) || a->q_len > 0, KVX_ERR_INVALID, "%s: v_norm needs q_len > 0", who);
  KVX_REQUIRE(!a->q_errors || (a->combination >= 0.0 && a->combination <= 1.0), KVX_ERR_INVALID,
              "%s: combination = %g, must be in [0, 1]", who, a->combination);
  return KVX_OK;
}

int kvx_h2o_update_select(const kvx_h2o_args* a, void* stream) {
  int rc = check_h2o(a, "kvx_h2o_update_select");
  if (rc != KVX_OK) return rc;
  return launch_h2o_update_select(*a, (hipStream_t)stream);
}

int kvx_h2o_update_select_static(const kvx_h2o_args* a, void* stream) {
  int rc = check_h2o(a, "kvx_h2o_update_select_static");
  if (rc != KVX_OK) return rc;
  return launch_h2o_update_select_static(*a, (hipStream_t)stream);
}

int kvx_sdpa_decode_h2o(const kvx_sdpa_args* a, const kvx_h2o_args* h, void* stream) {
  int rc = check_sdpa_common(a, "kvx_sdpa_decode_h2o", true);
  if (rc != KVX_OK) return rc;
  rc = check_h2o(h, "kvx_sdpa_decode_h2o");
  if (rc != KVX_OK) return rc;
  KVX_REQUIRE(a->q_len == 1, KVX_ERR_INVALID, "kvx_sdpa_decode_h2o: q_len must be 1, got %d", a->q_len);
  const int G = a->Hq / a->Hkv;
  KVX_REQUIRE(G >= 1 && G <= 16 && (G <= 8 || a->D <= 128), KVX_ERR_UNSUPPORTED, "kvx_sdpa_decode_h2o: group size %d not in 1 .. 16 (1 .. 8 with head size 256)", G);
  KVX_REQUIRE(!h->v_norm && !h->q_errors, KVX_ERR_UNSUPPORTED,
              "kvx_sdpa_decode_h2o: v_norm / q_errors policies take kvx_sdpa_decode + kvx_h2o_update_select");
  KVX_REQUIRE(h->k == 1 && h->kv_len == a->kv_len && h->B == a->B && h->Hkv == a->Hkv, KVX_ERR_INVALID,
              "kvx_sdpa_decode_h2o: needs k == 1 and the cache shape of the attention call");
  KVX_REQUIRE(aligned16(a->workspace), KVX_ERR_WORKSPACE, "kvx_sdpa_decode_h2o: workspace must be 16-byte aligned");
  KVX_REQUIRE(h->workspace && h->workspace_bytes >= h2o_workspace(*h), KVX_ERR_WORKSPACE, "kvx_sdpa_decode_h2o: h2o workspace of %zu bytes needed", h2o_workspace(*h));
  return launch_sdpa_decode(*a, h, (hipStream_t)stream);
}

int kvx_rmsnorm_rows(const void* x, int64_t x_row_stride, void* out, int64_t out_row_stride, const float* weight, int64_t rows,
                     int32_t dim, float eps, void* stream) {
  KVX_REQUIRE(rows >= 0 && dim > 0, KVX_ERR_INVALID, "kvx_rmsnorm_rows: rows=%lld, dim=%d", (long long)rows, dim);
  if (rows == 0) return KVX_OK;
  KVX_REQUIRE(x && out && weight, KVX_ERR_INVALID, "kvx_rmsnorm_rows: NULL pointer");
  KVX_REQUIRE(dim % 8 == 0 && dim <= 8192, KVX_ERR_UNSUPPORTED, "kvx_rmsnorm_rows: dim=%d must be a multiple of 8, at most 8192", dim);
  KVX_REQUIRE(aligned16(x) && aligned16(out) && aligned16(weight) && mult8(x_row_stride) && mult8(out_row_stride), KVX_ERR_INVALID,
              "kvx_rmsnorm_rows: rows must be 16-byte aligned");
  return launch_rmsnorm_rows(x, x_row_stride, out, out_row_stride, weight, rows, dim, eps, (hipStream_t)stream);
}

int kvx_add_rmsnorm_rows(const void* x, int64_t x_row_stride, const void* delta, int64_t delta_row_stride, void* x_out,
                         int64_t x_out_row_stride, void* out, int64_t out_row_stride, const float* weight, int64_t rows, int32_t dim,
                         float eps, void* stream) {
  KVX_REQUIRE(rows >= 0 && dim > 0, KVX_ERR_INVALID, "kvx_add_rmsnorm_rows: rows=%lld, dim=%d", (long long)rows, dim);
  if (rows == 0) return KVX_OK;
  KVX_REQUIRE(x && delta && x_out && out && weight, KVX_ERR_INVALID, "kvx_add_rmsnorm_rows: NULL pointer");
  KVX_REQUIRE(dim % 8 == 0 && dim <= 8192, KVX_ERR_UNSUPPORTED, "kvx_add_rmsnorm_rows: dim=%d must be a multiple of 8, at most 8192", dim);
  KVX_REQUIRE(aligned16(x) && aligned16(delta) && aligned16(x_out) && aligned16(out) && aligned16(weight) && mult8(x_row_stride) &&
                  mult8(delta_row_stride) && mult8(x_out_row_stride) && mult8(out_row_stride),
              KVX_ERR_INVALID, "kvx_add_rmsnorm_rows: rows must be 16-byte aligned");
  KVX_REQUIRE(out != x && out != delta, KVX_ERR_INVALID, "kvx_add_rmsnorm_rows: out must not alias the inputs");
  return launch_add_rmsnorm_rows(x, x_row_stride, delta, delta_row_stride, x_out, x_out_row_stride, out, out_row_stride, weight, rows, dim,
                                 eps, (hipStream_t)stream);
}

int kvx_swiglu_rows(const void* gate_up, int64_t gate_up_row_stride, void* out, int64_t out_row_stride, int64_t rows, int32_t dim,
                    void* stream) {
  KVX_REQUIRE(rows >= 0 && dim > 0, KVX_ERR_INVALID, "kvx_swiglu_rows: rows=%lld, dim=%d", (long long)rows, dim);
  if (rows == 0) return KVX_OK;
  KVX_REQUIRE(gate_up && out, KVX_ERR_INVALID, "kvx_swiglu_rows: NULL pointer");
  KVX_REQUIRE(dim % 8 == 0, KVX_ERR_UNSUPPORTED, "kvx_swiglu_rows: dim=%d must be a multiple of 8", dim);
  KVX_REQUIRE(aligned16(gate_up) && aligned16(out) && mult8(gate_up_row_stride) && mult8(out_row_stride) &&
                  gate_up_row_stride >= 2 * (int64_t)dim && out_row_stride >= dim,
              KVX_ERR_INVALID, "kvx_swiglu_rows: rows must be 16-byte aligned, gate_up rows 2 * dim long");
  KVX_REQUIRE(out != gate_up, KVX_ERR_INVALID, "kvx_swiglu_rows: out must not alias gate_up");
  return launch_swiglu_rows(gate_up, gate_up_row_stride, out, out_row_stride, rows, dim, (hipStream_t)stream);
}

int kvx_qk_norm_rope(void* qkv, int64_t stride_b, int64_t stride_t, int32_t B, int32_t num, int32_t Hq, int32_t Hkv, int32_t D,
                     const float* q_weight, const float* k_weight, float eps, const float* cos, const float* sin, int32_t table_rows,
                     int32_t input_pos, void* stream) {
  KVX_REQUIRE(B >= 0 && num >= 0 && Hq > 0 && Hkv > 0, KVX_ERR_INVALID, "kvx_qk_norm_rope: B=%d num=%d Hq=%d Hkv=%d", B, num, Hq, Hkv);
  if (B == 0 || num == 0) return KVX_OK;
  KVX_REQUIRE(D == 64 || D == 128 || D == 256, KVX_ERR_UNSUPPORTED, "kvx_qk_norm_rope: head size %d not in {64, 128, 256}", D);
  KVX_REQUIRE(qkv && cos && sin, KVX_ERR_INVALID, "kvx_qk_norm_rope: NULL pointer");
  KVX_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), KVX_ERR_INVALID, "kvx_qk_norm_rope: give both norm weights or none");
  KVX_REQUIRE(input_pos >= 0 && (int64_t)input_pos + num <= table_rows, KVX_ERR_INVALID,
              "kvx_qk_norm_rope: positions %d..%lld exceed the %d rows of the cos/sin tables", input_pos, (long long)input_pos + num - 1, table_rows);
  KVX_REQUIRE(stride_t >= (int64_t)(Hq + Hkv) * D, KVX_ERR_INVALID, "kvx_qk_norm_rope: token stride %lld shorter than the query and key heads",
              (long long)stride_t);
  KVX_REQUIRE(aligned16(qkv) && aligned16(cos) && aligned16(sin) && mult8(stride_b) && mult8(stride_t) &&
                  (!q_weight || (aligned16(q_weight) && aligned16(k_weight))),
              KVX_ERR_INVALID, "kvx_qk_norm_rope: pointers and strides must keep 16-byte alignment");
  return launch_qk_norm_rope(qkv, stride_b, stride_t, B, num, Hq, Hkv, D, q_weight, k_weight, eps, cos, sin, input_pos, (hipStream_t)stream);
}

}  // extern "C"
