// H2O score update and eviction choice for gfx950.
//
// Reference behaviour: keys_values/kvcache/h2o.py:146-199 (scores += weights, optional
// normalisation by residency) and keys_values/kvcache/attn_weights.py:771-783 (argsort / topk of
// the smallest scores). Output order here is ascending (value, slot), i.e. a stable argsort cut at k.
//
// Two shapes of the problem:
//   k == 1 (single-token decode): a streaming pass over all rows with many workgroups; each folds
//          its slice into one 64-bit key (ordered value bits << 32 | slot) and publishes it with
//          an integer atomicMin, which is order independent and therefore deterministic.
//   k  > 1 (chunked prefill): one workgroup per (batch, head) row. A 4-pass 8-bit radix select over
//          the ordered value bits finds the k-th smallest value; elements below it, plus the
//          lowest-slot elements equal to it, are gathered into LDS and bitonic-sorted as 64-bit
//          (value, slot) keys.
#include "kvx_common.h"

namespace kvx {
namespace {

constexpr int SEL_THREADS = 1024;
constexpr int MAX_K = 4096;

// Monotone map float -> uint32 (a < b  <=>  key(a) < key(b)); -0.0 is folded onto +0.0 first, as
// comparisons treat them as equal.
__device__ __forceinline__ uint32_t ordered_bits(float x) {
  x += 0.0f;
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Value the selection compares: the score, or the score divided by the slot's residency
// (keys_values/kvcache/h2o.py:183-196).
__device__ __forceinline__ float select_value(float score, const kvx_h2o_args& a, const int32_t* tp_row, int idx) {
  if (!a.normalize) return score;
  const int t = max(tp_row[idx], a.prefill_len - 1);
  return score / (float)(a.input_pos - t);
}

// ---- k == 1 ---------------------------------------------------------------------------------

__global__ void argmin_init_kernel(unsigned long long* best, int rows) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < rows) best[i] = ~0ull;
}

__global__ __launch_bounds__(256) void update_argmin_kernel(const kvx_h2o_args a, unsigned long long* best) {
  const int row = blockIdx.y;
  const int b = row / a.Hkv, hh = row % a.Hkv;
  float* sc = a.scores + b * a.sc_stride_b + hh * a.sc_stride_h;
  const float* w = a.w ? a.w + (int64_t)row * a.kv_len : nullptr;
  const int32_t* tpr = a.token_pos ? a.token_pos + b * a.tp_stride_b + hh * a.tp_stride_h : nullptr;
  unsigned long long mine = ~0ull;
  // 4 consecutive slots per lane per step, 4096 slots per workgroup
  const int base = blockIdx.x * 4096;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int i0 = base + it * 1024 + threadIdx.x * 4;
    if (i0 + 3 < a.kv_len && ((a.sc_stride_h | a.sc_stride_b) & 3) == 0) {
      f32x4_t s = *(const f32x4_t*)(sc + i0);
      if (w) {
        const f32x4_t ww = *(const f32x4_t*)(w + i0);  // rows of w are kv_len long: aligned only if kv_len % 4 == 0
        s += ww;
        *(f32x4_t*)(sc + i0) = s;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i0 + e < a.limit) {
          const unsigned long long key = ((unsigned long long)ordered_bits(select_value(s[e], a, tpr, i0 + e)) << 32) | (unsigned)(i0 + e);
          mine = key < mine ? key : mine;
        }
    } else {
      for (int e = 0; e < 4; ++e) {
        const int i = i0 + e;
        if (i >= a.kv_len) break;
        float s = sc[i];
        if (w) {
          s += w[i];
          sc[i] = s;
        }
        if (i < a.limit) {
          const unsigned long long key = ((unsigned long long)ordered_bits(select_value(s, a, tpr, i)) << 32) | (unsigned)i;
          mine = key < mine ? key : mine;
        }
      }
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const unsigned long long o = __shfl_xor(mine, off, 64);
    mine = o < mine ? o : mine;
  }
  __shared__ unsigned long long wbest[4];
  if ((threadIdx.x & 63) == 0) wbest[threadIdx.x >> 6] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long m = wbest[0];
    for (int i = 1; i < 4; ++i) m = wbest[i] < m ? wbest[i] : m;
    if (m != ~0ull) atomicMin(best + row, m);
  }
}

__global__ void argmin_finish_kernel(const unsigned long long* best, int32_t* next_index, int rows) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < rows) next_index[i] = (int32_t)(best[i] & 0xffffffffull);
}

// ---- k > 1 ----------------------------------------------------------------------------------

__global__ __launch_bounds__(SEL_THREADS) void update_select_kernel(const kvx_h2o_args a) {
  __shared__ unsigned long long cand[MAX_K];
  __shared__ uint32_t hist[256];
  __shared__ uint32_t wave_cnt[SEL_THREADS / 64];
  __shared__ uint32_t sh_prefix, sh_krem, sh_nless, sh_eqbase;

  const int tid = threadIdx.x;
  const int row = blockIdx.x;
  const int b = row / a.Hkv, hh = row % a.Hkv;
  float* sc = a.scores + b * a.sc_stride_b + hh * a.sc_stride_h;
  const float* w = a.w ? a.w + (int64_t)row * a.kv_len : nullptr;
  const int32_t* tpr = a.token_pos ? a.token_pos + b * a.tp_stride_b + hh * a.tp_stride_h : nullptr;

  // pass 0: scores += w. Every later pass of this thread touches the same slots it wrote here.
  if (w)
    for (int i = tid; i < a.kv_len; i += SEL_THREADS) sc[i] += w[i];

  int kpad = 1;
  while (kpad < a.k) kpad <<= 1;
  for (int i = tid; i < kpad; i += SEL_THREADS) cand[i] = ~0ull;
  if (tid == 0) {
    sh_prefix = 0;
    sh_krem = (uint32_t)a.k;
    sh_nless = 0;
    sh_eqbase = 0;
  }
  __syncthreads();

  // radix select: after the pass for digit `dg`, sh_prefix holds the digits dg..3 of the k-th
  // smallest key and sh_krem its rank among the keys sharing them.
  for (int dg = 3; dg >= 0; --dg) {
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    const uint32_t prefix = sh_prefix;
    const uint32_t himask = dg == 3 ? 0u : (0xffffffffu << (8 * (dg + 1)));
    for (int i = tid; i < a.limit; i += SEL_THREADS) {
      const uint32_t u = ordered_bits(select_value(sc[i], a, tpr, i));
      if ((u & himask) == prefix) atomicAdd(&hist[(u >> (8 * dg)) & 255u], 1u);
    }
    __syncthreads();
    if (tid == 0) {
      uint32_t krem = sh_krem, cum = 0;
      int d = 0;
      for (; d < 256; ++d) {
        if (cum + hist[d] >= krem) break;
        cum += hist[d];
      }
      sh_prefix = prefix | ((uint32_t)d << (8 * dg));
      sh_krem = krem - cum;
    }
    __syncthreads();
  }
  const uint32_t ustar = sh_prefix;   // k-th smallest value
  const uint32_t need_eq = sh_krem;   // how many slots equal to it are taken (lowest slots first)
  const uint32_t nless = (uint32_t)a.k - need_eq;

  // gather: slots below ustar in any order, slots equal to it by ascending slot
  const int lane = tid & 63, wave = tid >> 6;
  for (int i0 = 0; i0 < a.limit; i0 += SEL_THREADS) {
    const int i = i0 + tid;
    uint32_t u = 0xffffffffu;
    bool less = false, eq = false;
    if (i < a.limit) {
      u = ordered_bits(select_value(sc[i], a, tpr, i));
      less = u < ustar;
      eq = u == ustar;
    }
    if (less) {
      const uint32_t pos = atomicAdd(&sh_nless, 1u);
      cand[pos] = ((unsigned long long)u << 32) | (unsigned)i;
    }
    const unsigned long long eqm = __ballot(eq);
    if (lane == 0) wave_cnt[wave] = (uint32_t)__popcll(eqm);
    __syncthreads();
    if (eq) {
      uint32_t rank = sh_eqbase + (uint32_t)__popcll(eqm & ((1ull << lane) - 1ull));
      for (int ww = 0; ww < wave; ++ww) rank += wave_cnt[ww];
      if (rank < need_eq) cand[nless + rank] = ((unsigned long long)u << 32) | (unsigned)i;
    }
    __syncthreads();
    if (tid == 0) {
      uint32_t t = 0;
      for (int ww = 0; ww < SEL_THREADS / 64; ++ww) t += wave_cnt[ww];
      sh_eqbase += t;
    }
    __syncthreads();
  }

  // bitonic sort of kpad 64-bit keys
  for (int size = 2; size <= kpad; size <<= 1)
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int t = tid; t < kpad / 2; t += SEL_THREADS) {
        const int lo = 2 * t - (t & (stride - 1));
        const int hi = lo + stride;
        const bool up = (lo & size) == 0;
        const unsigned long long x = cand[lo], y = cand[hi];
        if ((x > y) == up) {
          cand[lo] = y;
          cand[hi] = x;
        }
      }
      __syncthreads();
    }
  for (int j = tid; j < a.k; j += SEL_THREADS) a.next_index[(int64_t)row * a.k + j] = (int32_t)(cand[j] & 0xffffffffull);
}

}  // namespace

size_t h2o_workspace(const kvx_h2o_args& a) { return a.k == 1 ? (size_t)a.B * a.Hkv * sizeof(unsigned long long) : 0; }

int launch_h2o_update_select(const kvx_h2o_args& a, hipStream_t st) {
  const int rows = a.B * a.Hkv;
  if (rows == 0) return KVX_OK;
  if (a.k == 1) {
    KVX_REQUIRE(a.workspace && a.workspace_bytes >= h2o_workspace(a), KVX_ERR_WORKSPACE,
                "kvx_h2o_update_select: workspace of %zu bytes needed", h2o_workspace(a));
    unsigned long long* best = (unsigned long long*)a.workspace;
    hipLaunchKernelGGL(argmin_init_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, best, rows);
    KVX_HIP(hipGetLastError());
    hipLaunchKernelGGL(update_argmin_kernel, dim3((a.kv_len + 4095) / 4096, rows), dim3(256), 0, st, a, best);
    KVX_HIP(hipGetLastError());
    hipLaunchKernelGGL(argmin_finish_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, best, a.next_index, rows);
    KVX_HIP(hipGetLastError());
    return KVX_OK;
  }
  hipLaunchKernelGGL(update_select_kernel, dim3(rows), dim3(SEL_THREADS), 0, st, a);
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

}  // namespace kvx
