// Single-token decode attention with per-key score-sums for gfx950 (HBM-bound).
//
// Reference behaviour: keys_values/attention/flashinfer_ops.py:193-275 (sdpa_decode: no mask, the
// weights divided by the group size), keys_values/csrc/kernels/sdpa_decode.cu:616-898 (the kernel
// it calls, which reads K and V once per QUERY head and keeps fp32 logits to turn them into
// weights afterwards, :838-854).
//
// Here one workgroup serves all G query heads of a (batch, KV head, split), so K and V cross HBM
// once, in one pass with both streams in flight: 8 or 16 lanes share a row (a lane owns 8 consecutive
// d, 16-byte loads, a wavefront instruction covers whole contiguous rows of K or V), the G logits of
// a row are v_dot2_f32_bf16 sums reduced over the row's lanes with DPP adds, and O += p V runs on
// the same lanes with dot2 over pairs of rows. Every row group of a wavefront keeps its own running
// maximum, sum and fp32 accumulator (the maximum moves lazily), so the loop has no barrier and no
// cross-lane traffic beyond the row reduction; groups and wavefronts are merged once at the end.
// The logits (log2 units) of a split are gathered in LDS, [key][head]. When a split's logits fit there
// (16384 / G keys for most shapes), they never leave the chip: a workgroup publishes its partial maximum and sum, waits
// until the other splits of its (batch, KV head) row have done the same (workgroups are dispatched in
// index order and a row's splits are neighbours, so they run at the same time; the wait is bounded),
// combines them into the row's base-2 log-sum-exp and turns its own logits into
// W = (1/G) sum_g exp2(logit_g - lse_g) on the spot; in the fused H2O form it also adds W to the cumulative
// scores and feeds the row's lowest-score slot. Longer splits, and a workgroup whose wait ran out, send the
// logits to an fp32 scratch in bursts of 32 KB (a write stream mixed into the reads costs HBM far more than
// its share of the bytes). One more launch follows the split kernel: some of its workgroups combine the splits'
// outputs, the others do the weights work of the splits that took the scratch route, and the one that finishes
// last publishes the chosen slots. K and V are touched once: they are loaded non-temporally. No float atomics
// anywhere.
// Quantised stores, and plain rows with 8 to 16 query heads per KV head, take a second form of the split kernel
// (decode_mfma_kernel, below) that does both products on the matrix cores: with codes to dequantise, or with that
// many dot products per loaded value, the form above is bound by its vector arithmetic, not by HBM.
#include "kvx_common.h"
#include <stdlib.h>

#include <atomic>
#include <mutex>

namespace kvx {
namespace {

constexpr int NTHREADS = 256;
constexpr int WAVES = 4;

struct DecodeParams {
  const uint16_t* q;
  const void* k;
  const void* v;
  const float* k_scale;
  const int32_t* k_zp;
  const float* v_scale;
  const int32_t* v_zp;
  uint16_t* o;
  float* lse_out;  // user (B, 1, Hq) or NULL
  float* w;        // user (B, Hkv, kv_len) or NULL
  float* logits;   // (B, Hkv, Tpad, G), G the padded group size
  float* part_o;   // (B, Hq, S, D)
  float* part_ml;  // (B, Hq, S, 2)
  unsigned long long* best;  // fused H2O form: (value, slot) minimum per (b, kvh) row, else NULL
  uint32_t* row_count;       // splits of a (b, kvh) row that have published their partial (resident form), then, in
                             // the fused H2O form, the row's workgroups of the tail kernel that have finished
  uint32_t* split_done;      // (B, Hkv, S): 1 where the split kernel itself turned its logits into weights
  uint32_t* tail_count;      // fused H2O form: workgroups of the tail kernel's second kind that have finished
  uint32_t* scratch_splits;  // caller's counter of the splits whose logits went through the scratch, or NULL
  int32_t qs_vec;            // quantiser state arrays are 16-byte aligned with strides that keep them so (vector loads of 4 keys)
  int32_t resident;          // the logits of a split stay in LDS
  int32_t spin_limit;        // polls of row_count before a workgroup gives up and sends its logits out
  int32_t poll_sleep;        // pause between two polls, in units of 512 cycles
  int32_t B, Hq, Hkv, kv_len, Tpad, num_splits, keys_per_split;
  int32_t Gr;  // query heads per KV head; the kernels' G is Gr rounded up to a power of two (heads Gr .. G - 1 are
               // dummies: zero queries, nothing of theirs is stored, their logits count for nothing)
  float c;
  int64_t q_sb, q_sh, k_sb, k_sh, k_st, v_sb, v_sh, v_st, o_sb, o_sh, qs_sb, qs_sh;
};


// Sum over the LPR lanes that share a row. Every lane of the group ends with the same bits: each
// step adds two values that the partner lane adds in the other order.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
template <int LPR>
__device__ __forceinline__ float row_group_sum(float x) {
  static_assert(LPR == 32 || LPR == 16 || LPR == 8, "row groups of 8, 16 or 32 lanes");
  if constexpr (LPR == 32) x += __shfl_xor(x, 16, 64);  // the other DPP row of the group
  if constexpr (LPR >= 16) {
    x = dpp_add<0x128>(x);  // row_ror:8
    x = dpp_add<0x124>(x);  // row_ror:4
  } else {
    x = dpp_add<0x141>(x);  // row_half_mirror
  }
  x = dpp_add<0x4E>(x);  // quad_perm [2,3,0,1]
  x = dpp_add<0xB1>(x);  // quad_perm [1,0,3,2]
  return x;
}

// Logits a workgroup holds in LDS: 64 KB where the merge buffer beside them is small enough for two workgroups
// per compute unit (what the registers allow), else 32 KB.
// Two workgroups per compute unit share 160 KB of LDS: the logits take what the merge buffer (4 G D floats) leaves of
// 80 KB, in whole pairs of steps of the widest kernel (256 keys).
constexpr int logit_floats(int G, int D) { return G * D <= 512 ? 16384 : (G * D <= 1024 ? (G == 16 ? 12288 : 14336) : 8192); }
constexpr int kCountStride = 64;  // a row's arrival counter has 256 bytes to itself: the polls of different rows go to different channels
constexpr float kNegBig = -1.0e30f;  // running maximum before the first key (finite: no inf - inf)
constexpr float kRescaleSlack = 8.0f;  // the running maximum moves only when a logit exceeds it by this

// Monotone map float -> uint32 (a < b  <=>  key(a) < key(b)); -0.0 is folded onto +0.0.
__device__ __forceinline__ uint32_t ordered_bits(float x) {
  x += 0.0f;
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Base-2 log-sum-exp of a query head from its splits' (maximum, sum) pairs, by one wavefront: lane s takes
// splits s, s + 64, ..., then butterflies; every lane returns the same bits. COHERENT: the pairs were
// written by other workgroups of the running kernel (device-coherent loads).
template <bool COHERENT>
__device__ __forceinline__ float row_lse(const float* part_ml, int num_splits, int lane) {
  const unsigned long long* ml = (const unsigned long long*)part_ml;
  float M = -INFINITY, L = 0.0f;
  for (int base = 0; base < num_splits; base += 64) {
    const int sp = base + lane;
    unsigned long long bits = 0xff800000ull;  // (maximum -inf, sum 0)
    if (sp < num_splits) bits = COHERENT ? __hip_atomic_load(ml + sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : ml[sp];
    const float m = __uint_as_float((uint32_t)bits), l = __uint_as_float((uint32_t)(bits >> 32));
    const float Mn = fmaxf(M, m);
    if (Mn > -INFINITY) L = L * fast_exp2(M - Mn) + l * fast_exp2(m - Mn);
    M = Mn;
  }
  float Mw = M;
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) Mw = fmaxf(Mw, __shfl_xor(Mw, off, 64));
  L = M > -INFINITY ? L * fast_exp2(M - Mw) : 0.0f;
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) L += __shfl_xor(L, off, 64);
  return Mw + fast_log2(L);
}

// The logits gathered in LDS leave as one contiguous burst (keys past the end of a chunk of CHUNK keys are -inf).
template <int G, int LGK, int CHUNK>
__device__ __forceinline__ void flush_logits(const float* lgbuf, float* lgrow, int lg_base, int k_end, int tid) {
  const int nkeys = min(LGK, (k_end - lg_base + CHUNK - 1) / CHUNK * CHUNK);
  f32x4_t* dst = (f32x4_t*)(lgrow + (int64_t)lg_base * G);
  for (int j = tid; j < nkeys * G / 4; j += NTHREADS) dst[j] = ((const f32x4_t*)lgbuf)[j];
}

// What a split does once its wavefronts have left their partial results in LDS (red: unnormalised outputs, rml:
// maximum and sum, per wavefront and head): combine them into the split's partial, and, in the resident form, wait
// for the row's other splits and turn this split's logits (lgbuf, [key][head]) into weights.
template <int D, int G, int LGK, int CHUNK>
__device__ __forceinline__ void finish_split(const DecodeParams& p, const kvx_h2o_args& hh, const int h2o, const float* lgbuf,
                                             const float (&red)[WAVES][G][D], const float (&rml)[WAVES][G][2], float* lgrow,
                                             const int lg_base, const int k_begin, const int k_end) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  __syncthreads();
  for (int i = tid; i < G * D; i += NTHREADS) {
    const int g = i / D, d = i % D;
    if (g >= p.Gr) continue;
    float M = rml[0][g][0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) M = fmaxf(M, rml[w][g][0]);
    float x = 0.0f, l = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float sc = fast_exp2(rml[w][g][0] - M);
      x += red[w][g][d] * sc;
      l += rml[w][g][1] * sc;
    }
    const int64_t o = ((int64_t)b * p.Hq + kvh * p.Gr + g) * p.num_splits + split;
    p.part_o[o * D + d] = x;
    if (d == 0) {
      // read by the row's other workgroups while this kernel runs: a device-coherent store
      const unsigned long long mlbits = ((unsigned long long)__float_as_uint(l) << 32) | __float_as_uint(M);
      __hip_atomic_store((unsigned long long*)(p.part_ml + o * 2), mlbits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (!lgrow || !p.resident) return;

  // ---- the row's log-sum-exp, and this split's logits into weights, without leaving the chip --------
  __shared__ float lse_sh[G];
  __shared__ int row_ready;
  __shared__ unsigned long long wbest[WAVES];
  const int row = b * p.Hkv + kvh;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the partial above has reached device-coherent memory
  __syncthreads();
  if (tid == 0) {
    uint32_t* cnt = p.row_count + row * kCountStride;
    __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    int ok = 0;
    for (int spin = 0; spin < p.spin_limit; ++spin) {  // bounded: a workgroup that gives up takes the scratch route
      if (__hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (uint32_t)p.num_splits) {
        ok = 1;
        break;
      }
      for (int z = 0; z < p.poll_sleep; ++z) __builtin_amdgcn_s_sleep(8);
    }
    row_ready = ok;
  }
  __syncthreads();
  if (!row_ready) {
    flush_logits<G, LGK, CHUNK>(lgbuf, lgrow, lg_base, k_end, tid);
    if (tid == 0) {
      p.split_done[(int64_t)row * p.num_splits + split] = 0u;
      if (p.scratch_splits) atomicAdd(p.scratch_splits, 1u);
    }
    return;
  }
  for (int g = wave; g < G; g += WAVES) {  // a wavefront per head: lane s takes splits s, s + 64, ...
    float lse = INFINITY;  // dummy heads: exp2(x - inf) = 0
    if (g < p.Gr) lse = row_lse<true>(p.part_ml + ((int64_t)b * p.Hq + kvh * p.Gr + g) * p.num_splits * 2, p.num_splits, lane);
    if (lane == 0) lse_sh[g] = lse;
  }
  __syncthreads();
  float lse[G];
#pragma unroll
  for (int g = 0; g < G; ++g) lse[g] = lse_sh[g];
  float* wr = p.w ? p.w + (int64_t)row * p.kv_len : nullptr;
  float* sc = h2o ? hh.scores + b * hh.sc_stride_b + kvh * hh.sc_stride_h : nullptr;
  const int32_t* tpr = (h2o && hh.token_pos) ? hh.token_pos + b * hh.tp_stride_b + kvh * hh.tp_stride_h : nullptr;
  const float inv_g = 1.0f / (float)p.Gr;
  unsigned long long mine = ~0ull;
  for (int k = k_begin + tid; k < k_end; k += NTHREADS) {
    const float* lg = lgbuf + (k - k_begin) * G;
    float acc = 0.0f;
#pragma unroll
    for (int g = 0; g < G; ++g) acc += fast_exp2(lg[g] - lse[g]);
    acc *= inv_g;
    if (wr) wr[k] = acc;
    if (h2o) {
      float val = sc[k] + acc;
      sc[k] = val;
      if (k < hh.limit) {
        if (hh.normalize) val = val / (float)(hh.input_pos - max(tpr[k], hh.prefill_len - 1));
        const unsigned long long key = ((unsigned long long)ordered_bits(val) << 32) | (unsigned)k;
        mine = key < mine ? key : mine;
      }
    }
  }
  if (h2o) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      const unsigned long long o = __shfl_xor(mine, off, 64);
      mine = o < mine ? o : mine;
    }
    if (lane == 0) wbest[wave] = mine;
    __syncthreads();
    if (tid == 0) {
      unsigned long long mn = wbest[0];
      for (int i = 1; i < WAVES; ++i) mn = wbest[i] < mn ? wbest[i] : mn;
      if (mn != ~0ull) atomicMin(p.best + row, mn);
    }
  }
  if (tid == 0) p.split_done[(int64_t)row * p.num_splits + split] = 1u;
}

template <int D, int G, int KV>
__global__ __launch_bounds__(NTHREADS) void decode_split_kernel(const DecodeParams p, const kvx_h2o_args hh, const int h2o) {
  constexpr bool F16 = kv_elem_f16(KV);  // element type of q, k, v, o
  constexpr int LPR = D / 8;     // lanes per row: a lane owns 8 consecutive d
  constexpr int RPI = 64 / LPR;  // rows per load instruction of a wavefront
  constexpr int U = 4;           // load instructions per step and tensor (even: rows pair up for dot2)
  constexpr int CH = U * RPI;    // keys per wavefront and step, contiguous
  constexpr int LGK = logit_floats(G, D) / G;  // keys whose logits are gathered in LDS before they go out in one burst
  __shared__ __align__(16) float lgbuf[LGK * G];  // [key][head]
  __shared__ float red[WAVES][G][D];
  __shared__ float rml[WAVES][G][2];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int kk = lane / LPR, dc = lane % LPR;
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int k_begin = split * p.keys_per_split;
  const int k_end = min(k_begin + p.keys_per_split, p.kv_len);

  uint32_t qv[G][4];  // bf16 pairs of q[head][8 dc .. 8 dc + 8]
#pragma unroll
  for (int g = 0; g < G; ++g) {
    u32x4_t t = {0u, 0u, 0u, 0u};
    if (g < p.Gr) t = *(const u32x4_t*)(p.q + b * p.q_sb + (int64_t)(kvh * p.Gr + g) * p.q_sh + 8 * dc);
#pragma unroll
    for (int e = 0; e < 4; ++e) qv[g][e] = t[e];
  }
  // Rows are addressed as a uniform base plus a 32-bit byte offset (the host checks the range). Plain rows only:
  // quantised stores take decode_mfma_kernel.
  static_assert(kv_is_plain(KV), "plain 16-bit rows");
  const uint8_t* kbase = (const uint8_t*)p.k + (b * p.k_sb + kvh * p.k_sh) * 2;
  const uint8_t* vbase = (const uint8_t*)p.v + (b * p.v_sb + kvh * p.v_sh) * 2;
  const uint32_t k_rowb = (uint32_t)p.k_st * 2, v_rowb = (uint32_t)p.v_st * 2, lane_off = 16 * dc;
  float* lgrow = p.logits ? p.logits + ((int64_t)b * p.Hkv + kvh) * p.Tpad * G : nullptr;
  int lg_base = k_begin;  // first key of the logits gathered in LDS

  // State of this lane's row group (rows kk, kk + RPI, ... of every chunk): identical in its lanes.
  float acc[G][8], m_run[G], l_run[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m_run[g] = kNegBig;
    l_run[g] = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[g][e] = 0.0f;
  }

  struct Rows {
    u32x4_t k[U], v[U];
  };
  // Rows past the end re-read the last valid row; their logits become -inf below.
  auto issue = [&](Rows& r, int chunk0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = min(chunk0 + u * RPI + kk, k_end - 1);
      r.k[u] = __builtin_nontemporal_load((const u32x4_t*)(kbase + ((uint32_t)key * k_rowb + lane_off)));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int key = min(chunk0 + u * RPI + kk, k_end - 1);
      r.v[u] = __builtin_nontemporal_load((const u32x4_t*)(vbase + ((uint32_t)key * v_rowb + lane_off)));
    }
  };
  auto consume = [&](Rows& r, int chunk0) {
    // logits (log2 units) of the U rows of this lane's group, all G heads
    float s[U][G];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const u32x4_t kx = r.k[u];
      const bool valid = chunk0 + u * RPI + kk < k_end;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float a = 0.0f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t kw = kx[e];  // a bit_cast applied to the vector element itself reads element 0
          a = dot2_acc<F16>(kw, qv[g][e], a);
        }
        a = row_group_sum<LPR>(a) * p.c;
        s[u][g] = valid ? a : -INFINITY;
      }
    }
    if (lgrow && dc == 0 && chunk0 < k_end) {
      typedef float fV __attribute__((ext_vector_type(G >= 4 ? 4 : G)));  // a key's G logits leave in one or two stores
      float* dst = lgbuf + (chunk0 - lg_base + kk) * G;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if constexpr (G == 1) {
          dst[u * RPI] = s[u][0];
        } else {
#pragma unroll
          for (int h = 0; h < G; h += 4) {
            fV t;
#pragma unroll
            for (int g = 0; g < (G >= 4 ? 4 : G); ++g) t[g] = s[u][h + g];
            *(fV*)(dst + u * RPI * G + h) = t;
          }
        }
      }
    }
    // running maximum: moved only when some logit of the wavefront exceeds it by the slack
    float smax[G];
    bool need = false;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mx = s[0][g];
#pragma unroll
      for (int u = 1; u < U; ++u) mx = fmaxf(mx, s[u][g]);
      smax[g] = mx;
      need |= mx > m_run[g] + kRescaleSlack;
    }
    if (__any(need)) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float mn = fmaxf(m_run[g], smax[g]);
        const float al = fast_exp2(m_run[g] - mn);
        m_run[g] = mn;
        l_run[g] *= al;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] *= al;
      }
    }
    // O += p V, two rows per dot2
#pragma unroll
    for (int u = 0; u < U; u += 2) {
      const u32x4_t xa = r.v[u], xb = r.v[u + 1];
      uint32_t pg[G];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float pa = fast_exp2(s[u][g] - m_run[g]);
        const float pb = fast_exp2(s[u + 1][g] - m_run[g]);
        l_run[g] += pa + pb;
        pg[g] = pack_pair<F16>(pa, pb);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t lo = __builtin_amdgcn_perm(xb[e], xa[e], 0x05040100u);
        const uint32_t hi = __builtin_amdgcn_perm(xb[e], xa[e], 0x07060302u);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          acc[g][2 * e] = dot2_acc<F16>(lo, pg[g], acc[g][2 * e]);
          acc[g][2 * e + 1] = dot2_acc<F16>(hi, pg[g], acc[g][2 * e + 1]);
        }
      }
    }
  };

  // Two steps in flight per wavefront: the loads of step i + 1 are issued before step i is consumed.
  const int nsteps = (k_end - k_begin + CH * WAVES - 1) / (CH * WAVES);
  const int stride = CH * WAVES;
  int chunk = k_begin + wave * CH;
  constexpr int FLUSH_STEPS = LGK / (CH * WAVES);
  static_assert(FLUSH_STEPS >= 2 && FLUSH_STEPS % 2 == 0, "the loop below advances two steps at a time");
  Rows ra, rb;
  issue(ra, chunk);
  for (int i = 0; i < nsteps; i += 2) {
    issue(rb, chunk + stride);
    __builtin_amdgcn_sched_barrier(0);
    consume(ra, chunk);
    __builtin_amdgcn_sched_barrier(0);  // the loads below reuse the registers consumed above
    issue(ra, chunk + 2 * stride);
    __builtin_amdgcn_sched_barrier(0);
    consume(rb, chunk + stride);
    __builtin_amdgcn_sched_barrier(0);
    chunk += 2 * stride;
    if (lgrow && !p.resident && ((i + 2) % FLUSH_STEPS == 0 || i + 2 >= nsteps)) {
      __syncthreads();
      flush_logits<G, LGK, CH>(lgbuf, lgrow, lg_base, k_end, tid);
      lg_base += LGK;
      __syncthreads();
    }
  }

  // ---- merge the RPI row groups of the wavefront, then the wavefronts, into one partial -----------
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float M = m_run[g];
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) M = fmaxf(M, __shfl_xor(M, off, 64));
    const float sc = fast_exp2(m_run[g] - M);
    float l = l_run[g] * sc;
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) l += __shfl_xor(l, off, 64);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float x = acc[g][e] * sc;
#pragma unroll
      for (int off = LPR; off < 64; off <<= 1) x += __shfl_xor(x, off, 64);
      if (lane < LPR) red[wave][g][lane * 8 + e] = x;
    }
    if (lane == 0) {
      rml[wave][g][0] = M;
      rml[wave][g][1] = l;
    }
  }
  finish_split<D, G, LGK, CH>(p, hh, h2o, lgbuf, red, rml, lgrow, lg_base, k_begin, k_end);
}

// ---- the same split with both products on the matrix cores --------------------------------------------------------
//
// For quantised stores and for more than four query heads per KV head the kernel above is bound by its vector
// arithmetic (G dot products per loaded pair of values on top of the dequantisation), not by HBM. Here the G heads are
// padded to the 16 columns of v_mfma_f32_16x16x32: S^T = K Q^T per 16 keys (the lane that holds key m of the tile
// loads 8 consecutive d of that row per matrix instruction: the row as it lies in memory is the A operand), then
// O^T += V^T P^T per 32 keys. The accumulator layout of S^T (lane = (head, keys 4 kg .. 4 kg + 3)) becomes the B
// operand of the second product without any exchange once the 32 keys of a block are taken in the order (tile 0:
// 4 kg .. 4 kg + 3, tile 1: 4 kg .. 4 kg + 3) per lane group kg; V^T is gathered to match: a lane loads, from each of
// its 8 keys, the D / 16 values of its d rows and regroups them (one byte permute per pair of bf16 values; for codes
// the regrouping is part of the dequantisation). What is left for the vector ALU is the dequantisation (3.5
// instructions per element, as the reference rounds) or half an instruction per V element, and the softmax of 16
// head columns per key. The running maximum is one per head (the four lane groups of a head column agree on it), it
// moves lazily as above. Everything after the key loop is shared with the kernel above.
template <bool F16>
__device__ __forceinline__ f32x4_t mfma_16x16x32(u32x4_t a, u32x4_t b, f32x4_t c) {
  if constexpr (F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  else return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// elem( (float)((int)code - zp) * scale ) for two codes with their own row state (two keys)
template <bool F16>
__device__ __forceinline__ uint32_t dequant_pair2(uint32_t c0, int32_t zp0, float sc0, uint32_t c1, int32_t zp1, float sc1) {
  return pack_pair<F16>((float)((int32_t)c0 - zp0) * sc0, (float)((int32_t)c1 - zp1) * sc1);
}

template <int D, int G, int KV>
__global__ __launch_bounds__(NTHREADS, D <= 128 ? 2 : 1) void decode_mfma_kernel(const DecodeParams p, const kvx_h2o_args hh, const int h2o) {
  constexpr bool F16 = kv_elem_f16(KV);
  constexpr bool U8 = !kv_is_plain(KV);  // codes + row state (8-bit or 4-bit store)
  constexpr bool U4 = kv_is_u4(KV);
  constexpr int KJ = D / 32;   // matrix instructions of the first product per 16-key tile
  constexpr int DPL = D / 16;  // d rows per lane = matrix instructions of the second product per 32-key block
  constexpr int CH = 32;       // keys per wavefront and step
  constexpr int NL4 = D >= 128 ? D / 128 : 1;                              // 4-bit rows: 16-byte loads per key of K
  constexpr int KR = U4 ? NL4 : (U8 ? D / 64 : KJ);                        // 16-byte loads per key of K
  constexpr int VW = U4 ? (DPL + 7) / 8 : (U8 ? (DPL + 3) / 4 : DPL / 2);  // dwords per key of V
  constexpr int LGK = logit_floats(G, D) / G;
  __shared__ __align__(16) float lgbuf[LGK * G];  // [key][head]
  __shared__ float red[WAVES][G][D];
  __shared__ float rml[WAVES][G][2];
  static_assert(D == 64 || D == 128 || (D == 256 && U8), "plain rows of 256 values take the vector-ALU kernel");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int m = lane & 15, kg = lane >> 4;
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int k_begin = split * p.keys_per_split;
  const int k_end = min(k_begin + p.keys_per_split, p.kv_len);

  // first d of the 8 this lane group supplies to matrix instruction e of the first product
  auto kslice = [&](int e) -> int {
    if constexpr (!U8) return 8 * (kg + 4 * e);
    else if constexpr (U4 && D == 64) return 8 * kg + 32 * e;
    else if constexpr (U4) return 16 * kg + 8 * (e & 1) + 64 * ((e >> 1) % NL4) + (D / 2) * (e / (2 * NL4));
    else return 16 * kg + 8 * (e & 1) + 64 * (e >> 1);
  };
  // d of row `mrow` of matrix instruction t of the second product
  auto dmap = [&](int t, int mrow) -> int {
    if constexpr (U4) return t < DPL / 2 ? (DPL / 2) * mrow + t : D / 2 + (DPL / 2) * mrow + (t - DPL / 2);
    else return DPL * mrow + t;
  };

  u32x4_t qb[KJ];  // B operands of the first product: head m (zero beyond the group), d slice of lane group kg
#pragma unroll
  for (int e = 0; e < KJ; ++e) {
    qb[e] = u32x4_t{0u, 0u, 0u, 0u};
    if (m < p.Gr) qb[e] = *(const u32x4_t*)(p.q + b * p.q_sb + (int64_t)(kvh * p.Gr + m) * p.q_sh + kslice(e));
  }
  constexpr int ES = U8 ? 1 : 2;
  const uint8_t* kbase = (const uint8_t*)p.k + (b * p.k_sb + kvh * p.k_sh) * ES;
  const uint8_t* vbase = (const uint8_t*)p.v + (b * p.v_sb + kvh * p.v_sh) * ES;
  const uint32_t k_rowb = (uint32_t)p.k_st * ES, v_rowb = (uint32_t)p.v_st * ES;
  const uint32_t k_lane = (U4 && D == 64) ? 8 * kg : 16 * kg;              // + 64 r for the r-th load of the row
  const uint32_t v_lane = (uint32_t)m * (U4 ? DPL / 2 : (U8 ? DPL : 2 * DPL));
  const int64_t qs_off = b * p.qs_sb + kvh * p.qs_sh;
  const char* ksb = (const char*)(p.k_scale + qs_off);
  const char* kzb = (const char*)(p.k_zp + qs_off);
  const char* vsb = (const char*)(p.v_scale + qs_off);
  const char* vzb = (const char*)(p.v_zp + qs_off);
  float* lgrow = p.logits ? p.logits + ((int64_t)b * p.Hkv + kvh) * p.Tpad * G : nullptr;
  int lg_base = k_begin;

  f32x4_t acc[DPL];
#pragma unroll
  for (int t = 0; t < DPL; ++t) acc[t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  float m_run = kNegBig, l_run = 0.0f;

  struct Rows {
    u32x4_t k[2][KR];
    float ks[2];
    int32_t kz[2];
    uint32_t v[8][VW];
    float vs[8];
    int32_t vz[8];
  };
  // Byte offsets of this lane's rows in the block at `chunk0`: K rows chunk0 + m and chunk0 + 16 + m, V rows
  // chunk0 + 4 kg (+ 0..3, + 16..19). A full block addresses them from two per-lane offsets that advance with the
  // block and multiples of the row stride; a block that reaches past the end clamps every key to the last valid row
  // (its logits become -inf below).
  const uint32_t k16 = 16u * k_rowb, v16 = 16u * v_rowb;
  auto load_k = [&](Rows& r, int gi, uint32_t off, int key) {
    const uint8_t* row = kbase + off;
#pragma unroll
    for (int x = 0; x < KR; ++x) {
      if constexpr (U4 && D == 64) {
        const u32x2_t c = __builtin_nontemporal_load((const u32x2_t*)row);
        r.k[gi][x] = u32x4_t{c[0], c[1], 0u, 0u};
      } else {
        r.k[gi][x] = __builtin_nontemporal_load((const u32x4_t*)(row + 64 * x));
      }
    }
    if constexpr (U8) {  // uniform base + 32-bit offset
      r.ks[gi] = *(const float*)(ksb + (uint32_t)key * 4u);
      r.kz[gi] = *(const int32_t*)(kzb + (uint32_t)key * 4u);
    }
  };
  auto load_v = [&](Rows& r, int j, uint32_t off) {
    const uint8_t* row = vbase + off;
    constexpr int BYTES = U4 ? DPL / 2 : (U8 ? DPL : 2 * DPL);  // this lane's share of the row
    if constexpr (BYTES == 16) {
      const u32x4_t x = __builtin_nontemporal_load((const u32x4_t*)row);
      r.v[j][0] = x[0]; r.v[j][1] = x[1]; r.v[j][2] = x[2]; r.v[j][3] = x[3];
    } else if constexpr (BYTES == 8) {
      const u32x2_t x = __builtin_nontemporal_load((const u32x2_t*)row);
      r.v[j][0] = x[0]; r.v[j][1] = x[1];
    } else if constexpr (BYTES == 4) {
      r.v[j][0] = __builtin_nontemporal_load((const uint32_t*)row);
    } else {
      static_assert(BYTES == 2, "4-bit rows of 64 values");
      r.v[j][0] = (uint32_t)__builtin_nontemporal_load((const uint16_t*)row);
    }
  };
  auto issue = [&](Rows& r, int chunk0) {
    if (chunk0 + CH <= k_end) {
      const uint32_t ko = (uint32_t)(chunk0 + m) * k_rowb + k_lane;
      load_k(r, 0, ko, chunk0 + m);
      load_k(r, 1, ko + k16, chunk0 + 16 + m);
      const int q0 = chunk0 + 4 * kg;
      if constexpr (U8) {
        if (p.qs_vec) {  // the four keys of a tile this lane group owns are neighbours: one 16-byte load each
#pragma unroll
          for (int gi = 0; gi < 2; ++gi) {
            const f32x4_t sc = *(const f32x4_t*)(vsb + (uint32_t)(q0 + 16 * gi) * 4u);
            const int4 zp = *(const int4*)(vzb + (uint32_t)(q0 + 16 * gi) * 4u);
            r.vs[4 * gi] = sc[0]; r.vs[4 * gi + 1] = sc[1]; r.vs[4 * gi + 2] = sc[2]; r.vs[4 * gi + 3] = sc[3];
            r.vz[4 * gi] = zp.x; r.vz[4 * gi + 1] = zp.y; r.vz[4 * gi + 2] = zp.z; r.vz[4 * gi + 3] = zp.w;
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            r.vs[j] = *(const float*)(vsb + (uint32_t)(q0 + 16 * (j >> 2) + (j & 3)) * 4u);
            r.vz[j] = *(const int32_t*)(vzb + (uint32_t)(q0 + 16 * (j >> 2) + (j & 3)) * 4u);
          }
        }
      }
      const uint32_t vo = (uint32_t)q0 * v_rowb + v_lane;
#pragma unroll
      for (int j = 0; j < 8; ++j) load_v(r, j, vo + (uint32_t)(j & 3) * v_rowb + (j >> 2) * v16);
    } else {
#pragma unroll
      for (int gi = 0; gi < 2; ++gi) {
        const int key = min(chunk0 + 16 * gi + m, k_end - 1);
        load_k(r, gi, (uint32_t)key * k_rowb + k_lane, key);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = min(chunk0 + 16 * (j >> 2) + 4 * kg + (j & 3), k_end - 1);
        if constexpr (U8) {
          r.vs[j] = *(const float*)(vsb + (uint32_t)key * 4u);
          r.vz[j] = *(const int32_t*)(vzb + (uint32_t)key * 4u);
        }
        load_v(r, j, (uint32_t)key * v_rowb + v_lane);
      }
    }
  };
  // A operand e of the first product for tile gi
  auto k_operand = [&](const Rows& r, int gi, int e) -> u32x4_t {
    if constexpr (!U8) {
      return r.k[gi][e];
    } else if constexpr (!U4) {
      const u32x4_t w = r.k[gi][e >> 1];
      return (e & 1) ? dequant_words<F16>(w[2], w[3], r.kz[gi], r.ks[gi]) : dequant_words<F16>(w[0], w[1], r.kz[gi], r.ks[gi]);
    } else {
      const u32x4_t w = r.k[gi][D >= 128 ? (e >> 1) % NL4 : 0];
      u32x2_t bytes;
      int shift;
      if constexpr (D >= 128) {
        bytes = (e & 1) ? u32x2_t{w[2], w[3]} : u32x2_t{w[0], w[1]};
        shift = (e / (2 * NL4)) ? 0 : 4;
      } else {
        bytes = u32x2_t{w[0], w[1]};
        shift = e ? 0 : 4;
      }
      const u32x2_t c = u4_codes(bytes, shift);
      return dequant_words<F16>(c[0], c[1], r.kz[gi], r.ks[gi]);
    }
  };
  // A operand t of the second product: value t of each of this lane's 8 keys, in key order
  auto v_operand = [&](const Rows& r, int t) -> u32x4_t {
    u32x4_t a;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int j0 = 2 * jj, j1 = 2 * jj + 1;
      if constexpr (!U8) {
        a[jj] = __builtin_amdgcn_perm(r.v[j1][t >> 1], r.v[j0][t >> 1], (t & 1) ? 0x07060302u : 0x05040100u);
      } else {
        uint32_t c0, c1;
        if constexpr (!U4) {
          c0 = (r.v[j0][t >> 2] >> (8 * (t & 3))) & 0xffu;
          c1 = (r.v[j1][t >> 2] >> (8 * (t & 3))) & 0xffu;
        } else {
          const int tb = t < DPL / 2 ? t : t - DPL / 2;  // byte of this lane's share; first half of the row: high nibble
          const int sh = 8 * (tb & 3) + (t < DPL / 2 ? 4 : 0);
          c0 = (r.v[j0][tb >> 2] >> sh) & 0xfu;
          c1 = (r.v[j1][tb >> 2] >> sh) & 0xfu;
        }
        a[jj] = dequant_pair2<F16>(c0, r.vz[j0], r.vs[j0], c1, r.vz[j1], r.vs[j1]);
      }
    }
    return a;
  };
  auto consume = [&](Rows& r, int chunk0) {
    f32x4_t s[2];
#pragma unroll
    for (int gi = 0; gi < 2; ++gi) {
      s[gi] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int e = 0; e < KJ; ++e) s[gi] = mfma_16x16x32<F16>(k_operand(r, gi, e), qb[e], s[gi]);
    }
    // this lane: head m, keys chunk0 + 16 gi + 4 kg + i (log2 units)
    float sv[8];
#pragma unroll
    for (int gi = 0; gi < 2; ++gi)
#pragma unroll
      for (int i = 0; i < 4; ++i) sv[4 * gi + i] = s[gi][i] * p.c;
    if (chunk0 + CH > k_end) {
#pragma unroll
      for (int gi = 0; gi < 2; ++gi)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (chunk0 + 16 * gi + 4 * kg + i >= k_end) sv[4 * gi + i] = -INFINITY;
    }
    if (lgrow && m < G && chunk0 < k_end) {
      float* dst = lgbuf + (chunk0 - lg_base + 4 * kg) * G + m;
#pragma unroll
      for (int gi = 0; gi < 2; ++gi)
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[(16 * gi + i) * G] = sv[4 * gi + i];
    }
    float mx = sv[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) mx = fmaxf(mx, sv[i]);
    if (__any(mx > m_run + kRescaleSlack)) {
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));  // the head's maximum over the four lane groups
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float mn = fmaxf(m_run, mx);
      const float al = fast_exp2(m_run - mn);
      m_run = mn;
      l_run *= al;
#pragma unroll
      for (int t = 0; t < DPL; ++t) acc[t] *= al;
    }
    float pv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pv[i] = fast_exp2(sv[i] - m_run);
      l_run += pv[i];
    }
    const u32x4_t pb = {pack_pair<F16>(pv[0], pv[1]), pack_pair<F16>(pv[2], pv[3]), pack_pair<F16>(pv[4], pv[5]), pack_pair<F16>(pv[6], pv[7])};
#pragma unroll
    for (int t = 0; t < DPL; ++t) acc[t] = mfma_16x16x32<F16>(v_operand(r, t), pb, acc[t]);
  };

  // Two steps in flight per wavefront: the loads of step i + 1 are issued before step i is consumed.
  const int nsteps = (k_end - k_begin + CH * WAVES - 1) / (CH * WAVES);
  const int stride = CH * WAVES;
  int chunk = k_begin + wave * CH;
  constexpr int FLUSH_STEPS = LGK / (CH * WAVES);
  static_assert(LGK % (CH * WAVES) == 0 && FLUSH_STEPS >= 2 && FLUSH_STEPS % 2 == 0, "the loop below advances two steps at a time");
  Rows ra, rb;
  issue(ra, chunk);
  for (int i = 0; i < nsteps; i += 2) {
    issue(rb, chunk + stride);
    __builtin_amdgcn_sched_barrier(0);
    consume(ra, chunk);
    __builtin_amdgcn_sched_barrier(0);  // the loads below reuse the registers consumed above
    issue(ra, chunk + 2 * stride);
    __builtin_amdgcn_sched_barrier(0);
    consume(rb, chunk + stride);
    __builtin_amdgcn_sched_barrier(0);
    chunk += 2 * stride;
    if (lgrow && !p.resident && ((i + 2) % FLUSH_STEPS == 0 || i + 2 >= nsteps)) {
      __syncthreads();
      flush_logits<G, LGK, CH>(lgbuf, lgrow, lg_base, k_end, tid);
      lg_base += LGK;
      __syncthreads();
    }
  }

  // ---- this wavefront's partial: sums over the four lane groups of a head, outputs by d ----------------------------
  float l = l_run;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (m < G) {
#pragma unroll
    for (int t = 0; t < DPL; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][m][dmap(t, 4 * kg + i)] = acc[t][i];
    if (kg == 0) {
      rml[wave][m][0] = m_run;
      rml[wave][m][1] = l;
    }
  }
  finish_split<D, G, LGK, CH>(p, hh, h2o, lgbuf, red, rml, lgrow, lg_base, k_begin, k_end);
}

// Before the split kernel: no split of a row has arrived, no row has a lowest-score slot yet.
__global__ void decode_init_kernel(uint32_t* row_count, unsigned long long* best, uint32_t* tail_count, int rows,
                                   uint32_t* scratch_splits, uint32_t scratch_splits_init) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < rows) {
    if (row_count) row_count[i * kCountStride] = 0u;
    if (best) best[i] = ~0ull;
  }
  if (i == 0 && tail_count) *tail_count = 0u;
  if (i == 0 && scratch_splits) *scratch_splits = scratch_splits_init;
}

// Combine the splits of one (b, query head): 4 groups of D threads each take a quarter of the
// splits, then the groups are added through LDS. Its first wavefront also produces the base-2 log-sum-exp.
template <int D, bool F16>
__device__ __forceinline__ void merge_job(const DecodeParams& p, const int bh) {
  __shared__ float red[4][D + 1];
  __shared__ float sM;
  const int b = bh / p.Hq, hqi = bh % p.Hq;
  const int d = threadIdx.x % D, grp = threadIdx.x / D;
  const float* ml = p.part_ml + (int64_t)bh * p.num_splits * 2;
  if (threadIdx.x < 64) {
    float mloc = -INFINITY;
    for (int s = threadIdx.x; s < p.num_splits; s += 64) mloc = fmaxf(mloc, ml[2 * s]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mloc = fmaxf(mloc, __shfl_xor(mloc, off, 64));
    if (threadIdx.x == 0) sM = mloc;
    // the log-sum-exp by the routine the split kernel uses for its own weights: the same bits on either route
    const float lse = row_lse<false>(ml, p.num_splits, threadIdx.x);
    if (threadIdx.x == 0 && p.lse_out) p.lse_out[bh] = lse;
  }
  __syncthreads();
  const float M = sM;
  float L = 0.0f, acc = 0.0f;
  for (int s = grp; s < p.num_splits; s += 4) {
    const float w = fast_exp2(ml[2 * s] - M);
    L += ml[2 * s + 1] * w;
    acc += p.part_o[((int64_t)bh * p.num_splits + s) * D + d] * w;
  }
  red[grp][d] = acc;
  if (d == 0) red[grp][D] = L;
  __syncthreads();
  if (grp == 0) {
    const float a4 = red[0][d] + red[1][d] + red[2][d] + red[3][d];
    const float l4 = red[0][D] + red[1][D] + red[2][D] + red[3][D];
    const float r = a4 / l4;
    const float other = __shfl_xor(r, 1, 64);
    if ((d & 1) == 0) *(uint32_t*)(p.o + b * p.o_sb + hqi * p.o_sh + d) = pack_pair<F16>(r, other);
  }
}

// W[b, kvh, k] = (1/G) sum_g exp2(logit[b, kvh, k, g] - lse[b, kvh*G+g]); one key per lane and pass,
// 4096 keys per workgroup of NT threads, for the splits whose logits went to the scratch (in the resident form:
// those whose wait ran out, normally none). With H2O set it also does the cache's score update and eviction choice
// in the same pass (keys_values/kvcache/h2o.py:175-196, keys_values/kvcache/attn_weights.py:773-774
// for one slot): scores += W, then the (value, slot) minimum of the row through an integer atomicMin; the workgroup
// that finishes last publishes the slot of every row's minimum. (That needs no fence: the minima and the count of
// finished workgroups are device-scope atomics, each waited for before the next; a release fence per workgroup
// would write the whole L2 back on this multi-die part.)
template <int G, bool H2O, int NT>
__device__ __forceinline__ void weights_job(const DecodeParams& p, const kvx_h2o_args& hh, const int bx, const int kvh, const int b, const int jobs) {
  typedef float fG __attribute__((ext_vector_type(G >= 4 ? 4 : (G == 2 ? 2 : 1))));
  constexpr int NV = G >= 4 ? G / 4 : 1;
  constexpr int PASSES = 4096 / NT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  __shared__ float lse_sh[G];
  __shared__ unsigned long long wbest[NT / 64];
  __shared__ int last_job;
  const uint32_t* done = p.resident ? p.split_done + ((int64_t)b * p.Hkv + kvh) * p.num_splits : nullptr;
  int pending = 1;
  if (done) {
    const int s0 = bx * 4096 / p.keys_per_split, s1 = min((bx * 4096 + 4095) / p.keys_per_split, p.num_splits - 1);
    pending = 0;
    for (int sp = s0 + tid; sp <= s1; sp += NT) pending |= done[sp] == 0u;
    pending = __syncthreads_or(pending);
  }
  unsigned long long mine = ~0ull;
  if (pending) {
    // the row's log-sum-exps from the splits' partials, by the routine the split kernel and the merge use
    for (int g = wave; g < G; g += NT / 64) {
      float l = INFINITY;  // dummy heads: exp2(x - inf) = 0
      if (g < p.Gr) l = row_lse<false>(p.part_ml + ((int64_t)b * p.Hq + kvh * p.Gr + g) * p.num_splits * 2, p.num_splits, lane);
      if (lane == 0) lse_sh[g] = l;
    }
    __syncthreads();
    float lse[G];
#pragma unroll
    for (int g = 0; g < G; ++g) lse[g] = lse_sh[g];
    const float* lgrow = p.logits + ((int64_t)b * p.Hkv + kvh) * p.Tpad * G;
    float* wr = p.w ? p.w + ((int64_t)b * p.Hkv + kvh) * p.kv_len : nullptr;
    float* sc = H2O ? hh.scores + b * hh.sc_stride_b + kvh * hh.sc_stride_h : nullptr;
    const int32_t* tpr = (H2O && hh.token_pos) ? hh.token_pos + b * hh.tp_stride_b + kvh * hh.tp_stride_h : nullptr;
    fG t[PASSES][NV];
#pragma unroll
    for (int it = 0; it < PASSES; ++it) {
      const int k = min(bx * 4096 + it * NT + tid, p.Tpad - 1);
#pragma unroll
      for (int j = 0; j < NV; ++j) t[it][j] = *((const fG*)(lgrow + (int64_t)k * G) + j);
    }
#pragma unroll
    for (int it = 0; it < PASSES; ++it) {
      const int k = bx * 4096 + it * NT + tid;
      if (k >= p.kv_len) break;
      if (done && done[k / p.keys_per_split]) continue;
      float acc = 0.0f;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float x;
        if constexpr (G >= 4) x = t[it][g / 4][g % 4];
        else if constexpr (G == 2) x = t[it][0][g];
        else x = t[it][0][0];
        acc += fast_exp2(x - lse[g]);
      }
      acc *= 1.0f / (float)p.Gr;
      if (wr) wr[k] = acc;
      if constexpr (H2O) {
        float val = sc[k] + acc;
        sc[k] = val;
        if (k < hh.limit) {
          if (hh.normalize) val = val / (float)(hh.input_pos - max(tpr[k], hh.prefill_len - 1));
          const unsigned long long key = ((unsigned long long)ordered_bits(val) << 32) | (unsigned)k;
          mine = key < mine ? key : mine;
        }
      }
    }
  }
  if constexpr (H2O) {
    if (pending) {
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) {
        const unsigned long long o = __shfl_xor(mine, off, 64);
        mine = o < mine ? o : mine;
      }
      if (lane == 0) wbest[wave] = mine;
      __syncthreads();
    }
    if (tid == 0) {
      if (pending) {
        unsigned long long mn = wbest[0];
        for (int i = 1; i < NT / 64; ++i) mn = wbest[i] < mn ? wbest[i] : mn;
        if (mn != ~0ull) {
          const unsigned long long old = __hip_atomic_fetch_min(p.best + b * p.Hkv + kvh, mn, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          asm volatile("s_waitcnt vmcnt(0)" : : "v"(old) : "memory");  // performed before this workgroup counts itself
        }
      }
      // counted per row first (the row's counter goes on from where the split kernel's arrivals left it), rows second:
      // no counter sees more than a few dozen increments
      const int wx = jobs / (p.B * p.Hkv);
      const uint32_t row_full = (p.resident ? (uint32_t)p.num_splits : 0u) + (uint32_t)wx - 1u;
      const bool row_last = __hip_atomic_fetch_add(p.row_count + (b * p.Hkv + kvh) * kCountStride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == row_full;
      last_job = row_last && __hip_atomic_fetch_add(p.tail_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (uint32_t)(p.B * p.Hkv - 1);
    }
    __syncthreads();
    if (last_job) {
      for (int i = tid; i < p.B * p.Hkv; i += NT)
        hh.next_index[i] = (int32_t)(__hip_atomic_load(p.best + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0xffffffffull);
    }
  }
}

// What follows the split kernel, in one launch: the first merge_jobs workgroups combine the splits of one (batch,
// query head) each; the others (MODE 1: weights wanted, MODE 2: fused H2O step) take 4096 keys of a (batch, KV head)
// row each. The two kinds do not depend on each other: both read what the split kernel left.
template <int D, bool F16, int G, int MODE>
__global__ __launch_bounds__(4 * D) void decode_tail_kernel(const DecodeParams p, const kvx_h2o_args hh, const int merge_jobs, const int wx) {
  if ((int)blockIdx.x < merge_jobs) {
    merge_job<D, F16>(p, blockIdx.x);
    return;
  }
  if constexpr (MODE > 0) {
    const int j = blockIdx.x - merge_jobs;
    weights_job<G, MODE == 2, 4 * D>(p, hh, j % wx, (j / wx) % p.Hkv, j / (wx * p.Hkv), (int)gridDim.x - merge_jobs);
  }
}

struct Plan {
  int G, num_splits, keys_per_split, Tpad, resident;
  size_t off_logits, off_part_o, off_part_ml, off_best, off_tail, off_count, off_done, total;
};

// Switches of the route the logits take, process-wide. Defaults come from the environment, read ONCE (first use):
// KVX_DECODE_RESIDENT=0 sends every split's logits through the scratch; KVX_DECODE_SPIN_LIMIT bounds the wait for a
// row's other splits in polls (0: no wait, every workgroup takes the scratch route); KVX_DECODE_POLL_SLEEP is the
// pause between two polls in units of 512 cycles. kvx_decode_tuning() replaces them at run time. Values are clamped:
// the longest wait a workgroup can spend is spin_limit x (poll_sleep x 512 + a load's latency) cycles, i.e.
// 2^20 x 64 x 512 cycles = 16 s at the clamps and about 30 ms at the defaults (2^15 polls, 4 x 512 cycles).
constexpr int kSpinDefault = 1 << 15, kSpinMax = 1 << 20, kSleepDefault = 4, kSleepMax = 64;
struct Tuning {
  std::atomic<int> resident{1}, spin_limit{kSpinDefault}, poll_sleep{kSleepDefault};
  int env_resident = 1, env_spin = kSpinDefault, env_sleep = kSleepDefault;
};
int clampi(int x, int lo, int hi) { return x < lo ? lo : (x > hi ? hi : x); }
int env_int(const char* name, int dflt) {
  const char* e = getenv(name);
  if (!e || !*e) return dflt;
  char* end = nullptr;
  const long v = strtol(e, &end, 10);
  return (end == e || *end) ? dflt : (int)(v < -1 ? -1 : (v > (1l << 30) ? (1l << 30) : v));  // not a number: the default
}
Tuning& tuning() {
  static Tuning t;
  static std::once_flag once;
  std::call_once(once, [] {
    t.env_resident = env_int("KVX_DECODE_RESIDENT", 1) != 0;
    t.env_spin = clampi(env_int("KVX_DECODE_SPIN_LIMIT", kSpinDefault), 0, kSpinMax);
    t.env_sleep = clampi(env_int("KVX_DECODE_POLL_SLEEP", kSleepDefault), 0, kSleepMax);
    t.resident = t.env_resident;
    t.spin_limit = t.env_spin;
    t.poll_sleep = t.env_sleep;
  });
  return t;
}

Plan make_plan(const kvx_sdpa_args& a, bool fused_h2o) {
  Plan pl;
  const int gr = a.Hq / a.Hkv;
  pl.G = gr <= 1 ? 1 : (gr <= 2 ? 2 : (gr <= 4 ? 4 : (gr <= 8 ? 8 : 16)));
  // One full round of workgroups (two per compute unit, what the registers allow) over the whole grid:
  // rows * kv_len / (2 CUs) keys per split, at least 256; with weights at most what the LDS holds of a split's
  // logits (a split that waits for its row holds its place, so the device then runs several rounds) and, LDS
  // permitting, at least kv_len / 128 (2 rows of 65536 keys: 45 us with 128 splits waiting for each other, 56 with 256).
  // Measured, with weights: 8 x 8 rows of 131072 keys, 4 rounds of 4096 keys beat 8 rounds of 2048 by 2 %; 8 rows of
  // 262144 keys take 182 us in one round of 4096 keys and 265 in four of 1024. Without weights: 32 rows of 262144
  // keys 631 us in 16 splits, 658 in 128; 8 rows of 16384 keys 22 us in 32 splits, 26 in 16 of 1024.
  const bool weights = a.w || fused_h2o;
  const int allow_resident = weights ? tuning().resident.load() : 0;
  const int lgk = logit_floats(pl.G, a.D) / pl.G;
  int splits = a.num_splits;
  if (splits <= 0) {
    int64_t keys = (int64_t)a.B * a.Hkv * a.kv_len / (2 * num_cus());
    if (keys < 256) keys = 256;
    if (allow_resident) {  // at most 128 splits wait for each other, unless the LDS limit asks for more
      if (keys < (a.kv_len + 127) / 128) keys = (a.kv_len + 127) / 128;
      if (keys > lgk) keys = lgk;
    }
    splits = (int)((a.kv_len + keys - 1) / keys);
  }
  splits = max(1, min(splits, 512));
  int kps = (a.kv_len + splits - 1) / splits;
  kps = ((kps + 63) / 64) * 64;  // keeps the chunks of a split aligned to the logits rows
  pl.keys_per_split = kps;
  pl.num_splits = (a.kv_len + kps - 1) / kps;
  pl.Tpad = ((a.kv_len + 63) / 64) * 64;
  size_t off = 0;
  pl.off_logits = off;
  off += weights ? (size_t)a.B * a.Hkv * pl.G * pl.Tpad * 4 : 0;
  pl.off_part_o = off;
  off += (size_t)a.B * a.Hq * pl.num_splits * a.D * 4;
  pl.off_part_ml = off;
  off += (size_t)a.B * a.Hq * pl.num_splits * 2 * 4;
  off = (off + 7) & ~(size_t)7;
  pl.off_best = off;
  off += fused_h2o ? (size_t)a.B * a.Hkv * 8 : 0;
  pl.off_tail = off;
  off += fused_h2o ? 8 : 0;
  pl.resident = allow_resident && kps <= lgk;
  off = (off + 255) & ~(size_t)255;
  pl.off_count = off;
  off += (pl.resident || fused_h2o) ? (size_t)a.B * a.Hkv * kCountStride * 4 : 0;
  pl.off_done = off;
  off += pl.resident ? (size_t)a.B * a.Hkv * pl.num_splits * 4 : 0;
  pl.total = (off + 255) & ~(size_t)255;
  return pl;
}

template <int D, bool F16, int G>
int launch_tail(const DecodeParams& p, const kvx_h2o_args* hh, hipStream_t st) {
  const int merge_jobs = p.B * p.Hq, wx = (p.kv_len + 4095) / 4096;
  const int weight_jobs = (hh || p.w) ? wx * p.Hkv * p.B : 0;
  const dim3 grid(merge_jobs + weight_jobs), block(4 * D);
  const kvx_h2o_args h2 = hh ? *hh : kvx_h2o_args{};
  if (hh) hipLaunchKernelGGL((decode_tail_kernel<D, F16, G, 2>), grid, block, 0, st, p, h2, merge_jobs, wx);
  else if (p.w) hipLaunchKernelGGL((decode_tail_kernel<D, F16, G, 1>), grid, block, 0, st, p, h2, merge_jobs, wx);
  else hipLaunchKernelGGL((decode_tail_kernel<D, F16, 1, 0>), grid, block, 0, st, p, h2, merge_jobs, wx);
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

// Three launches: the counters' reset (only when something counts), the split kernel, the tail.
template <int D, int G>
int launch_dg(const DecodeParams& p, int kv, const kvx_h2o_args* hh, hipStream_t st) {
  dim3 grid(p.num_splits, p.Hkv, p.B);
  const int rows = p.B * p.Hkv;
  if (p.resident || hh || p.scratch_splits) {
    // splits that take the scratch route by plan (the resident form switched off or too long for the LDS) count from the start
    const uint32_t by_plan = (p.logits && !p.resident) ? (uint32_t)(rows * p.num_splits) : 0u;
    hipLaunchKernelGGL(decode_init_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, (p.resident || hh) ? p.row_count : nullptr,
                       hh ? p.best : nullptr, hh ? p.tail_count : nullptr, rows, p.scratch_splits, by_plan);
    KVX_HIP(hipGetLastError());
  }
  const kvx_h2o_args h2 = hh ? *hh : kvx_h2o_args{};
  const int h2o = hh != nullptr;
  // quantised stores and groups of 8 heads or more: both products on the matrix cores
  {
    if (kv == KVX_KV_U4) hipLaunchKernelGGL((decode_mfma_kernel<D, G, KVX_KV_U4>), grid, dim3(NTHREADS), 0, st, p, h2, h2o);
    else if (kv == KVX_KV_U8) hipLaunchKernelGGL((decode_mfma_kernel<D, G, KVX_KV_U8>), grid, dim3(NTHREADS), 0, st, p, h2, h2o);
    else if (kv == KVX_KV_U4_F16) hipLaunchKernelGGL((decode_mfma_kernel<D, G, KVX_KV_U4_F16>), grid, dim3(NTHREADS), 0, st, p, h2, h2o);
    else if (kv == KVX_KV_U8_F16) hipLaunchKernelGGL((decode_mfma_kernel<D, G, KVX_KV_U8_F16>), grid, dim3(NTHREADS), 0, st, p, h2, h2o);
    else if constexpr (D <= 128 && G >= 8) {
      if (kv == KVX_KV_F16) hipLaunchKernelGGL((decode_mfma_kernel<D, G, KVX_KV_F16>), grid, dim3(NTHREADS), 0, st, p, h2, h2o);
      else hipLaunchKernelGGL((decode_mfma_kernel<D, G, KVX_KV_BF16>), grid, dim3(NTHREADS), 0, st, p, h2, h2o);
    }
  }
  if constexpr (G <= 8) {
    if (kv_is_plain(kv) && (D > 128 || G < 8)) {
      if (kv == KVX_KV_F16) hipLaunchKernelGGL((decode_split_kernel<D, G, KVX_KV_F16>), grid, dim3(NTHREADS), 0, st, p, h2, h2o);
      else hipLaunchKernelGGL((decode_split_kernel<D, G, KVX_KV_BF16>), grid, dim3(NTHREADS), 0, st, p, h2, h2o);
    }
  }
  KVX_HIP(hipGetLastError());
  return kv_elem_f16(kv) ? launch_tail<D, true, G>(p, hh, st) : launch_tail<D, false, G>(p, hh, st);
}

template <int D>
int launch_d(const DecodeParams& p, int G, int kv, const kvx_h2o_args* hh, hipStream_t st) {
  switch (G) {
    case 1: return launch_dg<D, 1>(p, kv, hh, st);
    case 2: return launch_dg<D, 2>(p, kv, hh, st);
    case 4: return launch_dg<D, 4>(p, kv, hh, st);
    case 8: return launch_dg<D, 8>(p, kv, hh, st);
    case 16:
      if constexpr (D <= 128) return launch_dg<D, 16>(p, kv, hh, st);
      break;
  }
  return set_error(KVX_ERR_UNSUPPORTED, "kvx_sdpa_decode: %d query heads per KV head (at most 16; at most 8 with head size 256)", p.Gr);
}

}  // namespace

size_t sdpa_decode_workspace(const kvx_sdpa_args& a, bool fused_h2o) { return make_plan(a, fused_h2o).total; }

void set_decode_tuning(int resident, int spin_limit, int poll_sleep) {
  Tuning& t = tuning();
  t.resident = resident < 0 ? t.env_resident : (resident != 0);
  t.spin_limit = spin_limit < 0 ? t.env_spin : clampi(spin_limit, 0, kSpinMax);
  t.poll_sleep = poll_sleep < 0 ? t.env_sleep : clampi(poll_sleep, 0, kSleepMax);
}

int launch_sdpa_decode(const kvx_sdpa_args& a, const kvx_h2o_args* hh, hipStream_t st) {
  const Plan pl = make_plan(a, hh != nullptr);
  KVX_REQUIRE(a.workspace && a.workspace_bytes >= pl.total, KVX_ERR_WORKSPACE,
              "kvx_sdpa_decode: workspace of %zu bytes needed, %zu given", pl.total, a.workspace_bytes);
  const int64_t es = kv_is_plain(a.kv_dtype) ? 2 : 1;
  KVX_REQUIRE((int64_t)a.kv_len * a.k_stride_t * es < (1ll << 32) && (int64_t)a.kv_len * a.v_stride_t * es < (1ll << 32), KVX_ERR_UNSUPPORTED,
              "kvx_sdpa_decode: one (batch, head) row set of K or V must span less than 4 GiB (kv_len %d, slot strides %lld / %lld)",
              a.kv_len, (long long)a.k_stride_t, (long long)a.v_stride_t);
  DecodeParams p;
  char* ws = (char*)a.workspace;
  p.q = (const uint16_t*)a.q;
  p.k = a.k;
  p.v = a.v;
  p.k_scale = a.k_scale; p.k_zp = a.k_zp; p.v_scale = a.v_scale; p.v_zp = a.v_zp;
  p.o = (uint16_t*)a.o;
  p.lse_out = a.lse;
  p.w = a.w;
  p.logits = (a.w || hh) ? (float*)(ws + pl.off_logits) : nullptr;
  p.part_o = (float*)(ws + pl.off_part_o);
  p.part_ml = (float*)(ws + pl.off_part_ml);
  p.best = hh ? (unsigned long long*)(ws + pl.off_best) : nullptr;
  p.tail_count = hh ? (uint32_t*)(ws + pl.off_tail) : nullptr;
  p.row_count = (uint32_t*)(ws + pl.off_count);
  p.split_done = (uint32_t*)(ws + pl.off_done);
  p.scratch_splits = a.decode_scratch_splits;
  p.resident = pl.resident;
  p.spin_limit = tuning().spin_limit.load();
  p.poll_sleep = tuning().poll_sleep.load();
  p.B = a.B; p.Hq = a.Hq; p.Hkv = a.Hkv; p.kv_len = a.kv_len; p.Tpad = pl.Tpad;
  p.Gr = a.Hq / a.Hkv;
  KVX_REQUIRE(p.Gr <= 16, KVX_ERR_UNSUPPORTED, "kvx_sdpa_decode: more than 16 query heads per KV head (%d)", p.Gr);
  p.qs_vec = (((uintptr_t)a.k_scale | (uintptr_t)a.k_zp | (uintptr_t)a.v_scale | (uintptr_t)a.v_zp) & 15) == 0 && a.qs_stride_b % 4 == 0 && a.qs_stride_h % 4 == 0;
  p.num_splits = pl.num_splits; p.keys_per_split = pl.keys_per_split;
  p.c = a.sm_scale * kLog2e;
  p.q_sb = a.q_stride_b; p.q_sh = a.q_stride_h;
  p.k_sb = a.k_stride_b; p.k_sh = a.k_stride_h; p.k_st = a.k_stride_t;
  p.v_sb = a.v_stride_b; p.v_sh = a.v_stride_h; p.v_st = a.v_stride_t;
  p.o_sb = a.o_stride_b; p.o_sh = a.o_stride_h;
  p.qs_sb = a.qs_stride_b; p.qs_sh = a.qs_stride_h;
  if (a.D == 128) return launch_d<128>(p, pl.G, a.kv_dtype, hh, st);
  if (a.D == 64) return launch_d<64>(p, pl.G, a.kv_dtype, hh, st);
  if (a.D == 256) return launch_d<256>(p, pl.G, a.kv_dtype, hh, st);
  return set_error(KVX_ERR_UNSUPPORTED, "kvx_sdpa_decode: head size %d not in {64, 128, 256}", a.D);
}

}  // namespace kvx
