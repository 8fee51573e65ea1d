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
//   k  > 1 (chunked prefill): one workgroup per (batch, head) row. The first pass adds the weights and
//          leaves the row's ordered value bits in LDS (rows of up to ~36K slots; longer rows are
//          re-read from global memory). A 4-pass 8-bit radix select finds the k-th smallest value;
//          elements below it, plus the lowest-slot elements equal to it, are gathered and
//          bitonic-sorted as 64-bit (value, slot) keys.
#include <mutex>

#include "kvx_common.h"

namespace kvx {
namespace {


// Monotone map float -> uint32 (a < b  <=>  key(a) < key(b)); -0.0 is folded onto +0.0 first, as
// comparisons treat them as equal.
__device__ __forceinline__ uint32_t ordered_bits(float x) {
  x += 0.0f;
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Value the selection compares: the score, or the score divided by the slot's residency
// (keys_values/kvcache/h2o.py:183-196).
__device__ __forceinline__ float residency_value(float score, const kvx_h2o_args& a, const int32_t* tp_row, int idx) {
  if (!a.normalize) return score;
  const int t = max(tp_row[idx], a.prefill_len - 1);
  return score / (float)(a.input_pos - t);
}

// Q-Hitter combination (keys_values/kvcache/qh2o.py:178-210): both terms are min-max normalised over
// all (head, slot < limit) entries of the batch element, then c*s + ((c-1)/2)*q + (1-c). Each
// product and sum is rounded on its own, as the reference's tensor expression is.
struct Modify {
  const float* qe;  // q_errors row, or nullptr: no modification
  float smin, sden, qmin, qden;
  float c, c2, c3;
};

// stats: 4 floats per (batch, head) row = min / max of the compared value and of q_errors.
__device__ __forceinline__ Modify load_modify(const kvx_h2o_args& a, const float* stats, int b, int hh) {
  Modify m;
  m.qe = nullptr;
  if (!stats) return m;
  m.qe = a.q_errors + b * a.sc_stride_b + hh * a.sc_stride_h;
  float smin = INFINITY, smax = -INFINITY, qmin = INFINITY, qmax = -INFINITY;
  for (int h = 0; h < a.Hkv; ++h) {
    const f32x4_t st = *(const f32x4_t*)(stats + ((int64_t)b * a.Hkv + h) * 4);
    smin = fminf(smin, st[0]);
    smax = fmaxf(smax, st[1]);
    qmin = fminf(qmin, st[2]);
    qmax = fmaxf(qmax, st[3]);
  }
  m.smin = smin;
  m.sden = smax - smin;
  m.qmin = qmin;
  m.qden = qmax - qmin;
  m.c = (float)a.combination;
  m.c2 = (float)((a.combination - 1.0) / 2.0);
  m.c3 = (float)(1.0 - a.combination);
  return m;
}

__device__ __forceinline__ float select_value(float score, const kvx_h2o_args& a, const int32_t* tp_row, int idx, const Modify& m) {
  float v = residency_value(score, a, tp_row, idx);
  if (m.qe) {
    const float s = (v - m.smin) / m.sden;
    const float q = (m.qe[idx] - m.qmin) / m.qden;
    v = __fadd_rn(__fadd_rn(__fmul_rn(m.c, s), __fmul_rn(m.c2, q)), m.c3);
  }
  return v;
}

// ---- policy variants: the accumulation pass ---------------------------------------------------

constexpr int SEL_THREADS = 1024;

// Deterministic workgroup reductions (wavefront butterfly, then the 16 partials in a fixed order).
template <typename Op>
__device__ __forceinline__ float block_reduce(float v, float* red, Op op) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = op(v, __shfl_xor(v, off, 64));
  __syncthreads();  // red may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = red[0];
  for (int i = 1; i < SEL_THREADS / 64; ++i) r = op(r, red[i]);
  return r;
}

// One workgroup per (batch, head) row: scores += instantaneous score, where the latter is w or,
// with v_norm, (v_norm*w / sum(v_norm*w)) * q_len (keys_values/kvcache/h2o.py:297-314); and the row's
// min / max of the compared value and of q_errors over the slots below limit, for the combination.
__global__ __launch_bounds__(SEL_THREADS) void accumulate_kernel(const kvx_h2o_args a, float* __restrict__ stats) {
  __shared__ float red[SEL_THREADS / 64];
  const int tid = threadIdx.x;
  const int row = blockIdx.x;
  const int b = row / a.Hkv, hh = row % a.Hkv;
  const int64_t off = b * a.sc_stride_b + hh * a.sc_stride_h;
  float* sc = a.scores + off;
  const float* w = a.w ? a.w + (int64_t)row * a.kv_len : nullptr;
  const float* vn = a.v_norm ? a.v_norm + off : nullptr;
  const float* qe = a.q_errors ? a.q_errors + off : nullptr;
  const int32_t* tpr = a.token_pos ? a.token_pos + b * a.tp_stride_b + hh * a.tp_stride_h : nullptr;
  float z = 1.0f;
  if (w && vn) {
    float part = 0.0f;
    for (int i = tid; i < a.kv_len; i += SEL_THREADS) part += vn[i] * w[i];
    z = block_reduce(part, red, [](float x, float y) { return x + y; });
  }
  const float ql = (float)a.q_len;
  float smin = INFINITY, smax = -INFINITY, qmin = INFINITY, qmax = -INFINITY;
  constexpr int PB = 4;
  for (int i0 = tid; i0 < a.kv_len; i0 += PB * SEL_THREADS) {
    float sv[PB], wv[PB], nv[PB], qv[PB];
#pragma unroll
    for (int j = 0; j < PB; ++j) {  // all loads of the batch before the first store (sc may alias for all the compiler knows)
      const int i = i0 + j * SEL_THREADS;
      const bool in = i < a.kv_len;
      sv[j] = in ? sc[i] : 0.0f;
      wv[j] = (in && w) ? w[i] : 0.0f;
      nv[j] = (in && w && vn) ? vn[i] : 0.0f;
      qv[j] = (qe && i < a.limit) ? qe[i] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < PB; ++j) {
      const int i = i0 + j * SEL_THREADS;
      if (i >= a.kv_len) break;
      float v = sv[j];
      if (w) {
        float inst = wv[j];
        if (vn) inst = __fmul_rn(__fmul_rn(nv[j], wv[j]) / z, ql);
        v = __fadd_rn(v, inst);
        sc[i] = v;
      }
      if (qe && i < a.limit) {
        const float cv = residency_value(v, a, tpr, i);
        smin = fminf(smin, cv);
        smax = fmaxf(smax, cv);
        qmin = fminf(qmin, qv[j]);
        qmax = fmaxf(qmax, qv[j]);
      }
    }
  }
  if (qe) {
    auto mn = [](float x, float y) { return fminf(x, y); };
    auto mx = [](float x, float y) { return fmaxf(x, y); };
    smin = block_reduce(smin, red, mn);
    smax = block_reduce(smax, red, mx);
    qmin = block_reduce(qmin, red, mn);
    qmax = block_reduce(qmax, red, mx);
    if (tid == 0) *(f32x4_t*)(stats + (int64_t)row * 4) = f32x4_t{smin, smax, qmin, qmax};
  }
}

// ---- k == 1 ---------------------------------------------------------------------------------

__global__ void argmin_init_kernel(unsigned long long* best, int rows) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < rows) best[i] = ~0ull;
}

__global__ __launch_bounds__(256) void update_argmin_kernel(const kvx_h2o_args a, unsigned long long* best, const float* stats) {
  const int row = blockIdx.y;
  const int b = row / a.Hkv, hh = row % a.Hkv;
  const Modify md = load_modify(a, stats, b, hh);
  float* sc = a.scores + b * a.sc_stride_b + hh * a.sc_stride_h;
  const float* w = a.w ? a.w + (int64_t)row * a.kv_len : nullptr;
  const int32_t* tpr = a.token_pos ? a.token_pos + b * a.tp_stride_b + hh * a.tp_stride_h : nullptr;
  unsigned long long mine = ~0ull;
  // 4 consecutive slots per lane per step, 4096 slots per workgroup
  const int base = blockIdx.x * 4096;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int i0 = base + it * 1024 + threadIdx.x * 4;
    // 16-byte loads need 16-byte aligned rows: the score rows by their strides, the rows of w (kv_len long) by kv_len
    if (i0 + 3 < a.kv_len && ((a.sc_stride_h | a.sc_stride_b) & 3) == 0 && (!w || (a.kv_len & 3) == 0)) {
      f32x4_t s = *(const f32x4_t*)(sc + i0);
      if (w) {
        const f32x4_t ww = *(const f32x4_t*)(w + i0);
        s += ww;
        *(f32x4_t*)(sc + i0) = s;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i0 + e < a.limit) {
          const unsigned long long key = ((unsigned long long)ordered_bits(select_value(s[e], a, tpr, i0 + e, md)) << 32) | (unsigned)(i0 + e);
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
          const unsigned long long key = ((unsigned long long)ordered_bits(select_value(s, a, tpr, i, md)) << 32) | (unsigned)i;
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

// CACHED: the row's ordered keys live in LDS after the first pass (rows of up to ~36K slots), so the
// radix passes and the gather never go back to global memory.
// Selections of more than MAX_PASS_K slots run as several launches: each takes the next a.k smallest
// (value, slot) keys above `bound` (the last key of the launch before, per row) and leaves its own last
// key there. out_off / out_stride place the launch's slots inside the row of next_index.
struct SelectPass {
  unsigned long long* bound;  // per row, or nullptr: a single launch
  int lower;                  // 1: only keys above bound[row] take part
  int out_off, out_stride;
};

template <bool CACHED>
__global__ __launch_bounds__(SEL_THREADS) void update_select_kernel(const kvx_h2o_args a, int kpad, const float* stats, const SelectPass ps) {
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  unsigned long long* cand = (unsigned long long*)dyn_lds;    // kpad entries
  uint32_t* keys = (uint32_t*)(dyn_lds + (size_t)kpad * 8);   // a.limit entries (CACHED only)
  __shared__ uint32_t hist[256];
  __shared__ uint32_t wave_cnt[SEL_THREADS / 64];
  __shared__ uint32_t sh_prefix, sh_krem, sh_diff;
  __shared__ int sh_hi;

  const int tid = threadIdx.x;
  const int row = blockIdx.x;
  const int b = row / a.Hkv, hh = row % a.Hkv;
  float* sc = a.scores + b * a.sc_stride_b + hh * a.sc_stride_h;
  const float* w = a.w ? a.w + (int64_t)row * a.kv_len : nullptr;
  const int32_t* tpr = a.token_pos ? a.token_pos + b * a.tp_stride_b + hh * a.tp_stride_h : nullptr;
  const Modify md = load_modify(a, stats, b, hh);
  // keys at or below the bound were taken by an earlier launch: they get the largest key and so never
  // come before a key still to be taken
  const unsigned long long bound = ps.lower ? ps.bound[row] : 0ull;
  const uint32_t bound_u = (uint32_t)(bound >> 32), bound_i = (uint32_t)bound;
  auto live_key = [&](float v, int i) -> uint32_t {
    const uint32_t u = ordered_bits(select_value(v, a, tpr, i, md));
    if (ps.lower && (u < bound_u || (u == bound_u && (uint32_t)i <= bound_i))) return 0xffffffffu;
    return u;
  };

  // pass 0: scores += w (every later pass of this thread touches the slots it wrote here) and the keys
  // One workgroup walks the whole row: batches of 8 loads per array are issued before anything is
  // stored, otherwise the stores to sc (which may alias w for all the compiler knows) serialise the
  // loads and the pass costs one memory round trip per element of a thread.
  const int n0 = max(a.kv_len, a.limit);
  constexpr int PB = 8;
  for (int i0 = tid; i0 < n0; i0 += PB * SEL_THREADS) {
    float sv[PB], wv[PB];
#pragma unroll
    for (int j = 0; j < PB; ++j) {
      const int i = i0 + j * SEL_THREADS;
      sv[j] = i < n0 ? sc[i] : 0.0f;
      wv[j] = (w && i < a.kv_len) ? w[i] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < PB; ++j) {
      const int i = i0 + j * SEL_THREADS;
      if (i >= n0) break;
      float v = sv[j];
      if (w && i < a.kv_len) {
        v += wv[j];
        sc[i] = v;
      }
      if (CACHED && i < a.limit) keys[i] = live_key(v, i);
    }
  }
  auto key_of = [&](int i) -> uint32_t {
    if constexpr (CACHED) return keys[i];
    else return live_key(sc[i], i);
  };

  for (int i = tid; i < kpad; i += SEL_THREADS) cand[i] = ~0ull;
  if (tid == 0) {
    sh_prefix = 0;
    sh_krem = (uint32_t)a.k;
    sh_diff = 0;
  }
  __syncthreads();

  // Bits that all keys of the row share need no pass, and skipping them matters: scores of one row
  // share their sign and most of their exponent, so a first digit taken from bit 31 down would send
  // nearly every key to the same few LDS counters (same-address atomics serialise).
  {
    const uint32_t key0 = key_of(0);
    uint32_t diff = 0;
    for (int i = tid; i < a.limit; i += SEL_THREADS) diff |= key_of(i) ^ key0;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) diff |= __shfl_xor(diff, off, 64);
    if ((tid & 63) == 0 && diff) atomicOr(&sh_diff, diff);
    __syncthreads();
    if (tid == 0) {
      const int top = sh_diff ? 32 - __clz(sh_diff) : 0;  // bits [0, top) differ somewhere
      sh_hi = top;
      sh_prefix = top >= 32 ? 0u : (key0 >> top) << top;
    }
    __syncthreads();
  }
  constexpr int RB = 8;
  // radix select over the remaining bits, 8 at a time from the top: after a pass sh_prefix holds the
  // bits [lo, 32) of the k-th smallest key and sh_krem its rank among the keys sharing them.
  for (int hi = sh_hi; hi > 0;) {
    const int lo = max(hi - 8, 0);
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    const uint32_t prefix = sh_prefix;
    const uint32_t himask = hi >= 32 ? 0u : (0xffffffffu << hi);
    const uint32_t dmask = (1u << (hi - lo)) - 1u;
    // keys are fetched eight at a time: a loop of one dependent LDS read per counter update would run at
    // the latency of that read
    for (int i0 = tid; i0 < a.limit; i0 += RB * SEL_THREADS) {
      uint32_t u[RB];
#pragma unroll
      for (int j = 0; j < RB; ++j) {
        const int i = i0 + j * SEL_THREADS;
        u[j] = i < a.limit ? key_of(i) : ~prefix;  // a key that cannot match the prefix
      }
#pragma unroll
      for (int j = 0; j < RB; ++j)
        if (i0 + j * SEL_THREADS < a.limit && (u[j] & himask) == prefix) atomicAdd(&hist[(u[j] >> lo) & dmask], 1u);
    }
    __syncthreads();
    if (tid < 64) {
      // the digit where the running count reaches the rank: 4 bins per lane, wavefront prefix sum
      const uint32_t krem = sh_krem;
      uint32_t h4[4], tot = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        h4[j] = hist[4 * tid + j];
        tot += h4[j];
      }
      uint32_t incl = tot;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const uint32_t o = __shfl_up(incl, off, 64);
        if (tid >= off) incl += o;
      }
      uint32_t cum = incl - tot;  // keys in the bins before this lane's
      if (cum < krem && incl >= krem) {
        int j = 0;
        for (; j < 3; ++j) {
          if (cum + h4[j] >= krem) break;
          cum += h4[j];
        }
        sh_prefix = prefix | ((uint32_t)(4 * tid + j) << lo);
        sh_krem = krem - cum;
      }
    }
    __syncthreads();
    hi = lo;
  }
  const uint32_t ustar = sh_prefix;   // k-th smallest value
  const uint32_t need_eq = sh_krem;   // how many slots equal to it are taken (lowest slots first)
  const uint32_t nless = (uint32_t)a.k - need_eq;

  // gather: slots below ustar, then slots equal to it by ascending slot. Every wavefront owns a
  // contiguous stretch of the row, so slot order is (wavefront, step, lane) order: one sweep counts
  // both kinds per wavefront, a prefix over the wavefronts gives each its places, a second sweep writes
  // them (no atomics, nothing a step has to wait for).
  const int lane = tid & 63, wave = tid >> 6;
  constexpr int NWV = SEL_THREADS / 64;
  __shared__ uint32_t wave_less[NWV];
  const int chunk = ((a.limit + NWV - 1) / NWV + 63) / 64 * 64;
  const int c_begin = wave * chunk, c_end = min(c_begin + chunk, a.limit);
  uint32_t my_less = 0, my_eq = 0;
  for (int i0 = c_begin; i0 < c_end; i0 += 64 * RB) {
    uint32_t u[RB];
#pragma unroll
    for (int j = 0; j < RB; ++j) {
      const int i = i0 + 64 * j + lane;
      u[j] = i < c_end ? key_of(i) : 0xffffffffu;
    }
#pragma unroll
    for (int j = 0; j < RB; ++j) {
      const bool in = i0 + 64 * j + lane < c_end;
      my_less += (uint32_t)__popcll(__ballot(in && u[j] < ustar));
      my_eq += (uint32_t)__popcll(__ballot(in && u[j] == ustar));
    }
  }
  if (lane == 0) {
    wave_less[wave] = my_less;
    wave_cnt[wave] = my_eq;
  }
  __syncthreads();
  uint32_t pos_less = 0, rank = 0;  // places taken by the wavefronts before this one
  for (int ww = 0; ww < wave; ++ww) {
    pos_less += wave_less[ww];
    rank += wave_cnt[ww];
  }
  const bool place_eq = rank < need_eq && my_eq;
  if (my_less || place_eq) {
    for (int i0 = c_begin; i0 < c_end; i0 += 64) {
      const int i = i0 + lane;
      const uint32_t u = i < c_end ? key_of(i) : 0xffffffffu;
      const bool less = i < c_end && u < ustar;
      const unsigned long long lm = __ballot(less);
      if (less) cand[pos_less + (uint32_t)__popcll(lm & ((1ull << lane) - 1ull))] = ((unsigned long long)u << 32) | (unsigned)i;
      pos_less += (uint32_t)__popcll(lm);
      if (place_eq) {
        const bool eq = i < c_end && u == ustar;
        const unsigned long long eqm = __ballot(eq);
        const uint32_t r = rank + (uint32_t)__popcll(eqm & ((1ull << lane) - 1ull));
        if (eq && r < need_eq) cand[nless + r] = ((unsigned long long)ustar << 32) | (unsigned)i;
        rank += (uint32_t)__popcll(eqm);
      }
    }
  }
  __syncthreads();

  // bitonic sort of kpad 64-bit keys. Comparator t of a stage with stride <= 64 only touches the 128
  // keys of its own wavefront's stretch, and a wavefront's LDS accesses execute in order: those
  // stages need no workgroup barrier.
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
      if (stride > 64 || (stride == 1 && 2 * size > 128)) __syncthreads();
      else __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    }
  __syncthreads();
  for (int j = tid; j < a.k; j += SEL_THREADS) a.next_index[(int64_t)row * ps.out_stride + ps.out_off + j] = (int32_t)(cand[j] & 0xffffffffull);
  if (ps.bound && tid == 0) ps.bound[row] = cand[a.k - 1];
}

}  // namespace

static bool is_variant(const kvx_h2o_args& a) { return a.v_norm != nullptr || a.q_errors != nullptr; }
constexpr int MAX_PASS_K = 4096;  // slots one launch of update_select_kernel sorts in LDS
// per row one 64-bit key: the running minimum of k == 1, or the bound handed from launch to launch when k > MAX_PASS_K
static size_t best_bytes(const kvx_h2o_args& a) {
  return (a.k == 1 || a.k > MAX_PASS_K) ? ((size_t)a.B * a.Hkv * sizeof(unsigned long long) + 15) / 16 * 16 : 0;
}

size_t h2o_workspace(const kvx_h2o_args& a) { return best_bytes(a) + (a.q_errors ? (size_t)a.B * a.Hkv * 4 * sizeof(float) : 0); }

int launch_h2o_update_select(const kvx_h2o_args& a_in, hipStream_t st) {
  kvx_h2o_args a = a_in;
  const int rows = a.B * a.Hkv;
  if (rows == 0) return KVX_OK;
  KVX_REQUIRE(h2o_workspace(a) == 0 || (a.workspace && a.workspace_bytes >= h2o_workspace(a)), KVX_ERR_WORKSPACE,
              "kvx_h2o_update_select: workspace of %zu bytes needed", h2o_workspace(a));
  float* stats = nullptr;
  if (is_variant(a)) {
    // the accumulation (and the batch statistics of the combination) first; what follows only selects
    if (a.q_errors) stats = (float*)((char*)a.workspace + best_bytes(a));
    if (a.w || stats) {
      hipLaunchKernelGGL(accumulate_kernel, dim3(rows), dim3(SEL_THREADS), 0, st, a, stats);
      KVX_HIP(hipGetLastError());
    }
    a.w = nullptr;
  }
  if (a.k == 1) {
    unsigned long long* best = (unsigned long long*)a.workspace;
    hipLaunchKernelGGL(argmin_init_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, best, rows);
    KVX_HIP(hipGetLastError());
    hipLaunchKernelGGL(update_argmin_kernel, dim3((a.kv_len + 4095) / 4096, rows), dim3(256), 0, st, a, best, (const float*)stats);
    KVX_HIP(hipGetLastError());
    hipLaunchKernelGGL(argmin_finish_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, best, a.next_index, rows);
    KVX_HIP(hipGetLastError());
    return KVX_OK;
  }
  // up to MAX_PASS_K slots per launch; a longer selection (the reference keeps the whole argsort when no chunk
  // size is set, keys_values/kvcache/attn_weights.py:773-774) continues above the last key of the launch before
  const int k_total = a.k;
  SelectPass ps;
  ps.bound = k_total > MAX_PASS_K ? (unsigned long long*)a.workspace : nullptr;
  ps.out_stride = k_total;
  for (int done = 0; done < k_total; done += MAX_PASS_K) {
    a.k = min(MAX_PASS_K, k_total - done);
    ps.lower = done > 0;
    ps.out_off = done;
    int kpad = 1;
    while (kpad < a.k) kpad <<= 1;
    // keys in LDS when the row fits beside the candidates (144 KB of the 160 KB of a compute unit)
    constexpr size_t kDynLimit = 144 * 1024;
    const size_t cached_bytes = (size_t)kpad * 8 + (size_t)a.limit * 4;
    if (cached_bytes <= kDynLimit) {
      if (cached_bytes > 48 * 1024)  // beyond the default dynamic LDS allowance (the setting is per device and kernel)
        KVX_HIP(hipFuncSetAttribute((const void*)update_select_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDynLimit));
      hipLaunchKernelGGL(update_select_kernel<true>, dim3(rows), dim3(SEL_THREADS), cached_bytes, st, a, kpad, (const float*)stats, ps);
    } else {
      hipLaunchKernelGGL(update_select_kernel<false>, dim3(rows), dim3(SEL_THREADS), (size_t)kpad * 8, st, a, kpad, (const float*)stats, ps);
    }
    KVX_HIP(hipGetLastError());
    a.w = nullptr;  // the scores are updated once
  }
  return KVX_OK;
}

// ---- the same call for callers that cannot allocate -------------------------------------------
//
// The workspace of the selection (the per-row 64-bit minimum keys of k == 1, the per-row statistics of
// the Q-Hitter combination) lives in a file-scope device array instead of caller memory. `scratch`
// is only a host-side stand-in for that array: its device address is looked up once per device with
// hipGetSymbolAddress (every device holds its own copy at its own address) and only that address is
// handed to kernels.
constexpr size_t kStaticScratchBytes = 128 * 1024;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

size_t h2o_static_scratch_bytes() { return kStaticScratchBytes; }

static int static_scratch_ptr(void** out) {
  static std::mutex mu;
  static void* ptrs[kMaxDevices] = {};
  int dev = 0;
  KVX_HIP(hipGetDevice(&dev));
  KVX_REQUIRE(dev >= 0 && dev < kMaxDevices, KVX_ERR_UNSUPPORTED, "kvx_h2o_update_select_static: device %d beyond the %d this library keeps scratch for", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    KVX_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    KVX_REQUIRE(p != nullptr, KVX_ERR_HIP, "kvx_h2o_update_select_static: no device address for the static scratch on device %d", dev);
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return KVX_OK;
}

int launch_h2o_update_select_static(const kvx_h2o_args& a_in, hipStream_t st) {
  kvx_h2o_args a = a_in;
  const size_t need = h2o_workspace(a);
  KVX_REQUIRE(need <= kStaticScratchBytes, KVX_ERR_WORKSPACE,
              "kvx_h2o_update_select_static: B * Hkv = %d rows need %zu bytes of scratch, the static array holds %zu", a.B * a.Hkv, need,
              kStaticScratchBytes);
  void* p = nullptr;
  const int rc = static_scratch_ptr(&p);
  if (rc != KVX_OK) return rc;
  a.workspace = p;
  a.workspace_bytes = kStaticScratchBytes;
  return launch_h2o_update_select(a, st);
}

}  // namespace kvx
