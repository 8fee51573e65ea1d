// Chunked-prefill attention for gfx950: O = softmax(s Q K^T + mask) V with the base-2 log-sum-exp.
//
// Reference behaviour: keys_values/attention/base.py:660-742 (eager arithmetic),
// keys_values/csrc/kernels/sdpa_prefill.cu:34-181 (what the FlashInfer prefill returns: O and
// base-2 LSE), keys_values/attention/attention_utils.py:238-247 (mask by token position).
//
// Work decomposition
//   The G query heads that share a KV head are packed into the row dimension: row r of a
//   (batch, KV head) pair is (query r / G, head r % G), R = q_len * G rows in all. A workgroup of
//   four (uint8 cache: eight) wavefronts owns 32 consecutive rows per wavefront and walks the key tiles of its KV
//   split, 64 keys at a time, so a K/V tile staged once in LDS serves all G heads.
//   Scores are produced TRANSPOSED, S^T = K Q^T (32x32x16 bf16 MFMA, keys along M, rows along N):
//   every lane then owns one row's statistics (running max and sum) and only the other half of the
//   wavefront holds the remaining keys of that row, so the online softmax needs a single
//   cross-lane exchange per tile. The accumulator layout of S^T is exactly the B-operand layout
//   of the second product O^T = V^T P^T once the 16 keys of a k-step are taken in the order
//   (0..3, 8..11 | 4..7, 12..15); the V^T operand is read from the row-major V tile with the
//   transposing LDS read (ds_read_b64_tr_b16), which delivers exactly that order.
//   K/V tiles travel global -> LDS by DMA (global_load_lds_dwordx4, no registers), double-buffered,
//   rows unpadded and XOR-swizzled against bank conflicts. The loop is software-pipelined: the
//   matrix cores add V(t-1) P(t-1) to O while the vector ALU turns S(t) into P(t).
#include <type_traits>
#include <utility>

#include "kvx_common.h"

namespace kvx {
namespace {

constexpr float kSlackLog2 = 8.0f;  // see the running-maximum update in the kernel

// Wavefronts per workgroup, 32 rows each. The uint8 cache takes 8: a tile is dequantised once per
// workgroup, so twice the rows halve that vector work per row (-13 % kernel time); for bf16 tiles the
// two sizes run alike and the smaller one leaves more workgroups for short chunks. At head size 256 the
// output accumulators (128 registers) leave no room for two wavefronts per SIMD: four for every store.
constexpr int nwaves(int kv, int D) { return (kv_is_plain(kv) || D > 128) ? 4 : 8; }  // kv: enum kvx_kv_dtype
constexpr int BN = 64;   // keys per tile

struct PrefillParams {
  const uint16_t* q;
  const void* k;
  const void* v;
  const float* k_scale;
  const int32_t* k_zp;
  const float* v_scale;
  const int32_t* v_zp;
  const int32_t* tp;
  uint16_t* o;
  float* lse;
  float* part_o;   // [split][group][R][D] fp32, unnormalised
  float* part_ml;  // [split][group][R][2]  (max in log2 units, sum)
  int32_t B, Hq, Hkv, G, q_len, kv_len, R, input_pos;
  int32_t num_splits, tiles_per_split, num_tiles, m_blocks;
  float c;  // sm_scale * log2(e)
  int64_t q_sb, q_sh, q_st, k_sb, k_sh, k_st, v_sb, v_sh, v_st, o_sb, o_sh, o_st;
  int64_t qs_sb, qs_sh, tp_sb, tp_sh;
};

// K and V tiles in LDS: [key][16-byte chunk], rows unpadded (D * 2 bytes), chunk c of row r stored at
// position c ^ key(r). Unpadded rows are what the global -> LDS DMA writes (a wavefront fills 1024
// contiguous bytes per instruction); the XOR then has to spread what one LDS phase touches over
// the 64 banks (256 bytes per cycle; measured on gfx950 with the LDS bank-conflict counter):
//   K, ds_read_b128:        16 consecutive rows, the same chunk      -> swz_k distinct over 16 rows
//   V, ds_read_b64_tr_b16:  half a wavefront reads 4 consecutive rows x 4 chunks (64 bytes a row): rows of 256
//                           bytes or more start at the same bank, so bits 2..3 of swz_v are distinct over r % 4
//                           (with bits 1..2, as for 128-byte rows, every such read took a 2-way conflict)
// Both depend on r % 16 only, so they repeat for the row groups a wavefront loads (16 or 32 rows apart).
template <int CPR>
__device__ __forceinline__ int swz_k(int r) { return CPR >= 16 ? (r & 15) : ((r >> 1) & 7); }
template <int CPR>
__device__ __forceinline__ int swz_v(int r) { return CPR >= 16 ? (((r & 3) << 2) | ((r >> 2) & 1)) : (((r & 3) << 1) | ((r >> 2) & 1)); }

template <int D>
struct alignas(16) Smem {
  static constexpr int CPR = D / 8;  // 16-byte chunks per row
  u32x4_t k[2][BN][CPR];
  u32x4_t v[2][BN][CPR];
  int32_t tp[2][BN];  // token positions of the K tile in the buffer of the same index
};

typedef short s16x4_t __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i (a = i % 4, r = i / 4) supplies the
// address of 4 consecutive bf16 of "row r, columns 4a..4a+3"; it receives column i of rows 0..3.
typedef char __attribute__((address_space(3))) * lds_ptr_t;
__device__ __forceinline__ u32x2_t lds_read_tr16(lds_ptr_t p) {
  const s16x4_t t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)(p));
  return __builtin_bit_cast(u32x2_t, t);
}


// Tile loader. A wavefront instruction covers RPW = 64 / CPR whole rows; wavefront w of the
// workgroup takes row groups w, w + 4, ... of the 64-row tile (NI groups each for K and for V).
// bf16 cache: DMA into LDS. uint8 cache: codes and row state go through registers (prefetched one
// tile ahead like the DMA), are dequantised to bf16 and written to the same LDS layout.
template <int D, int KV>
struct Loader {
  static constexpr bool U8 = !kv_is_plain(KV);  // codes through registers (8-bit or 4-bit store)
  static constexpr bool U4 = kv_is_u4(KV);
  static constexpr int CPR = D / 8;
  static constexpr int RPW = 64 / CPR;        // rows per wavefront instruction: 4 (D=128), 8 (D=64)
  static constexpr int NWAVES = nwaves(KV, D);
  static constexpr int NTHREADS = 64 * NWAVES;
  static constexpr int NI = BN / RPW / NWAVES;     // instructions per wavefront per operand: 4 / 2
  static constexpr int ESZ = U8 ? 1 : 2;
  // row groups of one wavefront are NWAVES RPW rows apart: with a multiple of 16 the XOR keys, and so
  // the source chunks, are the same for all of them (not for D = 256 with four wavefronts: 8 rows)
  static constexpr bool SAME_CHUNK = (NWAVES * RPW) % 16 == 0;
  const char* kbase;
  const char* vbase;
  const float* ks;
  const int32_t* kz;
  const float* vs;
  const int32_t* vz;
  const int32_t* tp;
  int64_t k_tile_bytes, v_tile_bytes, k_st, v_st;
  int wave, lane, kv_len, rl;
  int cgk[NI], cgv[NI];         // the source chunk that belongs at this lane's LDS position, per row group
  int shk[SAME_CHUNK ? 1 : NI], shv[SAME_CHUNK ? 1 : NI];  // 4-bit store: nibble of this lane's K / V chunk (4 = high)
  uint32_t lds_k, lds_v;        // LDS addresses of the K and V buffers (wavefront-uniform)
  uint32_t lds_kw, lds_vw;      // the same plus this wavefront's row-group offset
  uint32_t koffs[NI], voffs[NI];  // byte offset of this lane's chunk of row group i inside a tile
  // uint8 path staging registers
  u32x2_t kc[NI], vc[NI];
  float ksr[NI], vsr[NI];
  int32_t kzr[NI], vzr[NI];

  __device__ __forceinline__ int row_of(int i) const { return (NWAVES * i + wave) * RPW + rl; }
  // byte offset of chunk c (8 values) inside a row
  __device__ __forceinline__ static uint32_t chunk_off(int c) { return U4 ? u4_byte_off<D>(c) : (uint32_t)(c * 8 * ESZ); }

  __device__ __forceinline__ void init(const PrefillParams& p, Smem<D>& sm, int b, int kvh, int tid) {
    lds_k = __builtin_amdgcn_readfirstlane(lds_addr_of(&sm.k[0][0][0]));
    lds_v = __builtin_amdgcn_readfirstlane(lds_addr_of(&sm.v[0][0][0]));
    wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wavefront-uniform: keeps the LDS targets in scalar registers
    lane = tid & 63;
    rl = lane / CPR;  // row inside the group
    kv_len = p.kv_len;
    k_st = p.k_st;
    v_st = p.v_st;
    kbase = (const char*)p.k + (b * p.k_sb + kvh * p.k_sh) * ESZ;
    vbase = (const char*)p.v + (b * p.v_sb + kvh * p.v_sh) * ESZ;
    const int64_t so = b * p.qs_sb + kvh * p.qs_sh;
    ks = p.k_scale + so;
    kz = p.k_zp + so;
    vs = p.v_scale + so;
    vz = p.v_zp + so;
    tp = p.tp ? p.tp + b * p.tp_sb + kvh * p.tp_sh : nullptr;
    k_tile_bytes = (int64_t)BN * p.k_st * ESZ;
    v_tile_bytes = (int64_t)BN * p.v_st * ESZ;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int r = row_of(i);
      cgk[i] = (lane % CPR) ^ swz_k<CPR>(r);  // the chunk that belongs at LDS position lane % CPR of row r
      cgv[i] = (lane % CPR) ^ swz_v<CPR>(r);
      if (i == 0 || !SAME_CHUNK) {
        shk[SAME_CHUNK ? 0 : i] = u4_shift<D>(cgk[i]);
        shv[SAME_CHUNK ? 0 : i] = u4_shift<D>(cgv[i]);
      }
    }
    lds_kw = lds_k + (uint32_t)(wave * RPW * CPR * 16);
    lds_vw = lds_v + (uint32_t)(wave * RPW * CPR * 16);
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      koffs[i] = (uint32_t)(row_of(i) * p.k_st * ESZ + chunk_off(cgk[i]));
      voffs[i] = (uint32_t)(row_of(i) * p.v_st * ESZ + chunk_off(cgv[i]));
    }
  }

  // a full tile of the bf16 cache into buffer BUF: one scalar add (into M0) per DMA instruction
  template <bool IS_K, int BUF, int I = 0>
  __device__ __forceinline__ void issue_full(const char* tb) {
    dma16_at<(uint32_t)((BUF * BN + NWAVES * I * RPW) * CPR * 16)>(tb, IS_K ? koffs[I] : voffs[I], IS_K ? lds_kw : lds_vw);
    if constexpr (I + 1 < NI) issue_full<IS_K, BUF, I + 1>(tb);
  }
  template <bool IS_K, int BUF>
  __device__ __forceinline__ void issue_full(int tile) {
    issue_full<IS_K, BUF, 0>((IS_K ? kbase : vbase) + tile * (IS_K ? k_tile_bytes : v_tile_bytes));
  }

  template <bool IS_K>
  __device__ __forceinline__ void issue_one(Smem<D>& sm, int tile, int buf, int tid) {
    const int key0 = tile * BN;
    const int tpb = buf;
    if constexpr (!U8) {
      if (key0 + BN <= kv_len) {  // the common case: immediate LDS offsets, shared scalar base
        if (buf == 0) issue_full<IS_K, 0>(tile);
        else issue_full<IS_K, 1>(tile);
        issue_tp<IS_K>(sm, tile, tpb);
        return;
      }
    }
    const char* base = IS_K ? kbase : vbase;
    const int64_t st = IS_K ? k_st : v_st;
    const char* tb = base + tile * (IS_K ? k_tile_bytes : v_tile_bytes);
    if (key0 + BN <= kv_len) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        if constexpr (!U8) {
          const uint32_t dst = (IS_K ? lds_k : lds_v) + (uint32_t)((buf * BN + (NWAVES * i + wave) * RPW) * CPR * 16);
          dma16(tb, IS_K ? koffs[i] : voffs[i], dst);
        } else {
          const int key = key0 + row_of(i);
          const u32x2_t c = *(const u32x2_t*)(tb + (IS_K ? koffs[i] : voffs[i]));
          if (IS_K) { kc[i] = c; ksr[i] = ks[key]; kzr[i] = kz[key]; }
          else { vc[i] = c; vsr[i] = vs[key]; vzr[i] = vz[key]; }
        }
      }
    } else {
      // last, partial tile: rows past the end re-read the last valid row (finite data); their
      // position is INT_MAX, so they are masked for every query and contribute exactly zero
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int key = min(key0 + row_of(i), kv_len - 1);
        const uint32_t off = (uint32_t)((int64_t)(key - key0) * st * ESZ) + chunk_off(IS_K ? cgk[i] : cgv[i]);
        if constexpr (!U8) {
          const uint32_t dst = (IS_K ? lds_k : lds_v) + (uint32_t)((buf * BN + (NWAVES * i + wave) * RPW) * CPR * 16);
          dma16(tb, off, dst);
        } else {
          const u32x2_t c = *(const u32x2_t*)(tb + off);
          if (IS_K) { kc[i] = c; ksr[i] = ks[key]; kzr[i] = kz[key]; }
          else { vc[i] = c; vsr[i] = vs[key]; vzr[i] = vz[key]; }
        }
      }
    }
    issue_tp<IS_K>(sm, tile, tpb);
  }

  // a full tile, not the last one of the walk: no bounds to check (bf16 tiles only)
  template <bool IS_K, int BUF>
  __device__ __forceinline__ void issue_steady(Smem<D>& sm, int tile) {
    static_assert(!U8, "codes go through registers");
    issue_full<IS_K, BUF>(tile);
    if (IS_K && tp && wave == 0)
      dma4((const char*)(tp + tile * BN), (uint32_t)lane * 4, __builtin_amdgcn_readfirstlane(lds_addr_of(&sm.tp[BUF][0])));
  }
  __device__ __forceinline__ void land_steady(Smem<D>& sm, int tile, int buf, int tid) {
    if (!tp && tid < BN) sm.tp[buf][tid] = tile * BN + tid;
  }

  // token positions of the K tile: one 4-byte DMA per lane of wavefront 0 (slots past the end
  // re-read the last valid one and are overwritten with INT_MAX when the tile lands)
  template <bool IS_K>
  __device__ __forceinline__ void issue_tp(Smem<D>& sm, int tile, int buf) {
    if (IS_K && tp && wave == 0) {
      const int key0 = tile * BN;
      const uint32_t dst = lds_addr_of(&sm.tp[buf][0]);
      dma4((const char*)(tp + key0), (uint32_t)min(lane, kv_len - 1 - key0) * 4, __builtin_amdgcn_readfirstlane(dst));
    }
  }

  // make tile `tile`, issued last, visible in LDS (called after s_waitcnt vmcnt(0), before the
  // barrier that publishes it)
  template <bool IS_K>
  __device__ __forceinline__ void land(Smem<D>& sm, int tile, int buf, int tid) {
    const int tpb = buf;
    if constexpr (U8) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int r = row_of(i);
        u32x2_t c = IS_K ? kc[i] : vc[i];
        if constexpr (U4) c = u4_codes(c, IS_K ? shk[SAME_CHUNK ? 0 : i] : shv[SAME_CHUNK ? 0 : i]);
        if (IS_K) sm.k[buf][r][lane % CPR] = dequant_words<kv_elem_f16(KV)>(c[0], c[1], kzr[i], ksr[i]);
        else sm.v[buf][r][lane % CPR] = dequant_words<kv_elem_f16(KV)>(c[0], c[1], vzr[i], vsr[i]);
      }
    }
    if (IS_K && tid < BN) {
      const int key = tile * BN + tid;
      if (!tp) sm.tp[tpb][tid] = key < kv_len ? key : INT_MAX;
      else if (key >= kv_len) sm.tp[tpb][tid] = INT_MAX;
    }
  }
};

template <int D, int KV>
__global__ __launch_bounds__(64 * nwaves(KV, D), (kv_is_plain(KV) && D <= 128) ? 2 : 1) void sdpa_prefill_kernel(const PrefillParams p) {
  constexpr bool F16 = kv_elem_f16(KV);  // element type of q, k, v, o
  constexpr int BM = 32 * nwaves(KV, D);  // rows per workgroup
  constexpr int CPR = D / 8;
  constexpr int KS = D / 16;  // k-steps of the first product
  constexpr int DT = D / 32;  // d tiles of the second product
  __shared__ Smem<D> sm;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n = lane & 31;  // row (query) owned by this lane within the wavefront's 32 rows
  const int h = lane >> 5;  // which half of each 8-wide k group / which 4-row group of the MFMA output

  const int group = blockIdx.x;  // b * Hkv + kvh: fastest-varying so that a KV head stays on one XCD
  const int mblk = blockIdx.y;
  const int split = blockIdx.z;
  const int b = group / p.Hkv;
  const int kvh = group % p.Hkv;

  const int row0w = mblk * BM + wave * 32;
  const int row = row0w + n;
  const bool row_ok = row < p.R;
  const int rowc = row_ok ? row : p.R - 1;
  const int qi = rowc / p.G;
  const int g = rowc % p.G;
  const int qpos = p.input_pos + qi;
  const int qpos_min_w = p.input_pos + min(row0w, p.R - 1) / p.G;

  // Q fragments (B operand): lane holds row n, d = 16 j + 8 h .. +8
  u32x4_t qf[KS];
  {
    const uint16_t* qp = p.q + b * p.q_sb + (int64_t)(kvh * p.G + g) * p.q_sh + (int64_t)qi * p.q_st;
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      u32x4_t t = row_ok ? *(const u32x4_t*)(qp + 16 * j + 8 * h) : u32x4_t{0, 0, 0, 0};
      qf[j] = t;
    }
  }

  // LDS byte offsets of this lane's operand fragments inside a tile buffer.
  // K (A operand of S^T = K Q^T): row 32 mt + n, chunk 2 j + h, stored at position chunk ^ swz_k(row).
  uint32_t ka[KS];
#pragma unroll
  for (int j = 0; j < KS; ++j) ka[j] = (uint32_t)(n * CPR + ((2 * j + h) ^ swz_k<CPR>(n))) * 16;
  // V (A operand of O^T = V^T P^T) through the transposing read: in its group of 16 lanes this lane
  // points at key row (i / 4) + 4 h of the 16-key block and at d columns 16 * (group % 2) + 4 (i % 4) .. +3
  // of the 32-d tile; the second read of a k-step is 8 rows further down (same XOR key, same positions).
  const int li = lane & 15;
  const int vrow = (li >> 2) + 4 * h;                              // + 32 mt + 16 j (+ 8)
  const int vcol = 16 * ((lane >> 4) & 1) + 4 * (li & 3);          // + 32 dt, bf16 elements
  uint32_t va[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int c = (32 * dt + vcol) >> 3;
    va[dt] = (uint32_t)((vrow * CPR + (c ^ swz_v<CPR>(vrow))) * 16 + (vcol & 7) * 2);
  }

  const int tile_begin = split * p.tiles_per_split;
  int tile_end = min(tile_begin + p.tiles_per_split, p.num_tiles);
  if (!p.tp) {
    // slots hold positions 0, 1, 2, ...: tiles past the last position any row of this workgroup may
    // see are masked out completely (the upper triangle of a causal first chunk) and are skipped
    const int qpos_max = p.input_pos + min(mblk * BM + BM - 1, p.R - 1) / p.G;
    tile_end = min(tile_end, qpos_max / BN + 1);
    if (tile_end <= tile_begin) {  // whole split invisible: an empty partial (only with num_splits > 1)
      if (row_ok) {
        const int64_t prow = ((int64_t)split * p.B * p.Hkv + group) * p.R + row;
        float* po = p.part_o + prow * D;
        const f32x4_t z = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int a = 0; a < 4; ++a) *(f32x4_t*)(po + dt * 32 + 8 * a + 4 * h) = z;
        if (h == 0) {
          p.part_ml[prow * 2] = -INFINITY;
          p.part_ml[prow * 2 + 1] = 0.0f;
        }
      }
      return;
    }
  }

  f32x16_t o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.0f;
  float m = -INFINITY;  // reference (lazy running maximum) of the raw, unscaled scores of this row
  const float slack = kSlackLog2 / p.c;
  float l = 0.0f;       // this lane's share of the running sum

  // S^T of one tile from the K tile in k[buf]: two independent accumulator chains
  auto qk = [&](f32x16_t (&s)[2], int buf) {
    const char* kb = (const char*)&sm.k[buf][0][0];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[mt][i] = 0.0f;
#pragma unroll
    for (int j = 0; j < KS; ++j)
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const u32x4_t kk = *(const u32x4_t*)(kb + ka[j] + mt * 32 * CPR * 16);
        s[mt] = mfma_32x32x16<F16>(kk, qf[j], s[mt]);
      }
  };
  // mask (only tiles that hold a position some row of this wavefront may not see)
  auto mask = [&](f32x16_t (&s)[2], int buf) {
    const int tpl = sm.tp[buf][lane];
    // bit k: key k of the tile holds a position some row of this wavefront may not see. In a cache with
    // scattered slots nearly every tile has a few such keys: only their groups of 8 keys are masked.
    const unsigned long long hidden = __ballot(tpl > qpos_min_w);
    if (hidden) {
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          if ((hidden >> (mt * 32 + 8 * a)) & 0xffull) {
            const int4 tq = *(const int4*)&sm.tp[buf][mt * 32 + 8 * a + 4 * h];
            if (tq.x > qpos) s[mt][4 * a + 0] = -INFINITY;
            if (tq.y > qpos) s[mt][4 * a + 1] = -INFINITY;
            if (tq.z > qpos) s[mt][4 * a + 2] = -INFINITY;
            if (tq.w > qpos) s[mt][4 * a + 3] = -INFINITY;
          }
        }
    }
  };

  // second product for one tile: O^T += V^T P^T with V from v[buf]; matrix instructions FIRST ..
  // FIRST + COUNT - 1 of the 4 DT in (key block, d tile) order
  auto pv_part = [&](const uint32_t (&pb)[2][8], int buf, auto first_tag, auto count_tag) {
    constexpr int FIRST_I = decltype(first_tag)::value, COUNT = decltype(count_tag)::value;
    // one LDS pointer per d tile; every read below is that pointer plus a compile-time offset
    lds_ptr_t vl[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vl[dt] = (lds_ptr_t)((const char*)&sm.v[buf][0][0] + va[dt]);
#pragma unroll
    for (int i = FIRST_I; i < FIRST_I + COUNT; ++i) {
      const int mt = i / (2 * DT), j = (i / DT) % 2, dt = i % DT;
      const u32x4_t pf = u32x4_t{pb[mt][4 * j], pb[mt][4 * j + 1], pb[mt][4 * j + 2], pb[mt][4 * j + 3]};
      const int rb = (32 * mt + 16 * j) * CPR * 16;
      const u32x2_t lo = lds_read_tr16(vl[dt] + rb);
      const u32x2_t hi = lds_read_tr16(vl[dt] + rb + 8 * CPR * 16);
      o[dt] = mfma_32x32x16<F16>(u32x4_t{lo[0], lo[1], hi[0], hi[1]}, pf, o[dt]);
    }
  };
  auto pv = [&](const uint32_t (&pb)[2][8], int buf) {
    pv_part(pb, buf, std::integral_constant<int, 0>{}, std::integral_constant<int, 4 * DT>{});
  };
  // The first NPRE matrix instructions of the second product go out right behind the first product:
  // they keep the matrix core busy while the vector ALU reduces the maximum of S(t), which has to wait
  // for the first product anyway.
  constexpr int NPRE = DT;

  // Pipeline: iteration t multiplies S(t) = K(t) Q^T, then lets the matrix cores add V(t-1) P(t-1)
  // to O while the vector ALU turns S(t) into P(t). K(t) sits in k[t & 1]; V(t-1) in v[(t-1) & 1];
  // K(t+1) and V(t) are in flight to the other buffers and are published by the barrier that ends
  // the iteration.
  Loader<D, KV> ld;
  ld.init(p, sm, b, kvh, tid);
  uint32_t pbs[2][2][8];  // packed P of the tile in buffer 0 / 1: written by one step, multiplied by the next
  // every split owns at least one tile (the host sizes the splits that way)
  ld.template issue_one<true>(sm, tile_begin, 0, tid);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the first K tile and the Q fragments have arrived
  ld.template land<true>(sm, tile_begin, 0, tid);
  __syncthreads();
  // one pipeline step; the first one has no previous tile to multiply
  // one pipeline step on the tile in buffer CUR (compile time: LDS offsets become immediates and P
  // alternates between two register sets instead of being copied)
  auto step = [&](auto first_tag, auto cur_tag, auto steady_tag, int t) {
    constexpr bool FIRST = decltype(first_tag)::value;
    constexpr int cur = decltype(cur_tag)::value;
    // STEADY: tiles t and t + 1 are full and tile t + 1 belongs to this walk
    constexpr bool STEADY = decltype(steady_tag)::value && kv_is_plain(KV);
    uint32_t (&pb_prev)[2][8] = pbs[cur ^ 1];
    uint32_t (&pb)[2][8] = pbs[cur];
    const bool has1 = STEADY || t + 1 < tile_end;
    if constexpr (STEADY) {
      ld.template issue_steady<false, cur>(sm, t);
      ld.template issue_steady<true, cur ^ 1>(sm, t + 1);
    } else {
      ld.template issue_one<false>(sm, t, cur, tid);
      if (has1) ld.template issue_one<true>(sm, t + 1, cur ^ 1, tid);
    }
    f32x16_t s[2];
    // Issue priority rises through the tile (0 for the first product, 1 for the dependent chain mask ->
    // maximum -> rescaling decision, 2 for the exponentials beside the second product, 3 for the way to the
    // barrier): of the two wavefronts on a SIMD the one closer to its barrier goes first, so the four
    // wavefronts of a workgroup wait less for each other. Measured -3 to -5 % on the kernel.
    __builtin_amdgcn_s_setprio(0);
    qk(s, cur);
    if constexpr (!FIRST) {
      pv_part(pb_prev, cur ^ 1, std::integral_constant<int, 0>{}, std::integral_constant<int, NPRE>{});
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_setprio(1);
    mask(s, cur);
    // ---- running maximum; rescale only when some row of the wavefront has a new maximum ------
    float mx = fmaxf(s[0][0], s[1][0]);
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(fmaxf(mx, s[0][i]), s[1][i]);
    mx = max_halves(mx);
    float alpha = 1.0f;
    // m is a reference, not the exact maximum: it moves only when a score exceeds it by 2^kSlackLog2
    // in the exponent, which keeps every p below 2^kSlackLog2 and makes rescaling rare
    const bool resc = __any(mx > m + slack);
    if (resc) {
      const float m_new = fmaxf(m, mx);
      const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
      alpha = fast_exp2((m - m_use) * p.c);
      l *= alpha;
      m = m_new;
    }
    // ---- O += V(t-1) P(t-1) on the matrix cores, P(t) = exp2(c S(t) - c m) on the vector ALU ----
    __builtin_amdgcn_s_setprio(2);
    if constexpr (!FIRST) pv_part(pb_prev, cur ^ 1, std::integral_constant<int, NPRE>{}, std::integral_constant<int, 4 * DT - NPRE>{});
    const float mc = (m == -INFINITY) ? 0.0f : m * p.c;
    float rs0 = 0.0f, rs1 = 0.0f;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float p0 = fast_exp2(fmaf(s[mt][i], p.c, -mc));
        const float p1 = fast_exp2(fmaf(s[mt][i + 1], p.c, -mc));
        rs0 += p0;
        rs1 += p1;
        pb[mt][i >> 1] = pack_pair<F16>(p0, p1);
      }
    l += rs0 + rs1;
    if constexpr (!FIRST) {
      // interleave in the instruction stream: each matrix instruction of the second product is
      // followed by the two LDS reads of the next one and by its share of the softmax arithmetic,
      // so the vector ALU works in the shadow of the matrix core instead of after it
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);  // operands of the first two go out ahead
      constexpr int NREST = 4 * DT - NPRE;
      constexpr int NV = (80 + NREST - 1) / NREST;  // VALU per matrix instruction: 80 per tile (fma, add, cvt)
      constexpr int NX = (32 + NREST - 1) / NREST;  // transcendental: 32 exp2 per tile
#pragma unroll
      for (int i = 0; i < NREST; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // 1 MFMA
        __builtin_amdgcn_sched_group_barrier(0x002, (NV + 1) / 2, 0);  // half of its vector work,
        __builtin_amdgcn_sched_group_barrier(0x400, (NX + 1) / 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);             // the 2 LDS reads of the next one,
        __builtin_amdgcn_sched_group_barrier(0x002, NV / 2, 0);        // the other half
        __builtin_amdgcn_sched_group_barrier(0x400, NX / 2, 0);
      }
      // keep the softmax arithmetic in this block: without a use here the optimiser sinks it
      // past the barrier below, out of the matrix core's shadow
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("" : "+v"(pb[mt][i]));
      asm volatile("" : "+v"(l));
      if (resc) {  // O (now including tile t-1) moves to the new reference maximum
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
      }
    }
    // ---- publish the tiles that were in flight -------------------------------------------------
    __builtin_amdgcn_s_setprio(3);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's DMA / loads have landed
    if constexpr (STEADY) {
      ld.land_steady(sm, t + 1, cur ^ 1, tid);
    } else {
      ld.template land<false>(sm, t, cur, tid);
      if (has1) ld.template land<true>(sm, t + 1, cur ^ 1, tid);
    }
    __syncthreads();
  };
  constexpr std::integral_constant<int, 0> B0{};
  constexpr std::integral_constant<int, 1> B1{};
  constexpr std::true_type YES{};
  constexpr std::false_type NO{};
  step(YES, B0, NO, tile_begin);
  int t = tile_begin + 1;
  // tiles whose successor is a full tile of this walk take the step without bounds checks
  const int steady_end = min(tile_end - 1, p.kv_len / BN - 1);  // t < steady_end: tiles t, t + 1 full, t + 1 < tile_end
  for (; t + 1 < steady_end; t += 2) {
    step(NO, B1, YES, t);
    step(NO, B0, YES, t + 1);
  }
  for (; t + 1 < tile_end; t += 2) {
    step(NO, B1, NO, t);
    step(NO, B0, NO, t + 1);
  }
  if (t < tile_end) {
    step(NO, B1, NO, t);
    pv(pbs[1], 1);
  } else {
    pv(pbs[0], 0);
  }

  // ---- epilogue -----------------------------------------------------------------------------
  const float lt = sum_halves(l);
  if (p.num_splits == 1) {
    const float inv = lt > 0.0f ? 1.0f / lt : 0.0f;
    if (row_ok) {
      uint16_t* op = p.o + b * p.o_sb + (int64_t)(kvh * p.G + g) * p.o_sh + (int64_t)qi * p.o_st;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          u32x2_t w2;
          w2[0] = pack_pair<F16>(o[dt][4 * a] * inv, o[dt][4 * a + 1] * inv);
          w2[1] = pack_pair<F16>(o[dt][4 * a + 2] * inv, o[dt][4 * a + 3] * inv);
          *(u32x2_t*)(op + dt * 32 + 8 * a + 4 * h) = w2;
        }
      if (p.lse && h == 0) p.lse[((int64_t)b * p.q_len + qi) * p.Hq + kvh * p.G + g] = m * p.c + fast_log2(lt);
    }
  } else {
    if (row_ok) {
      const int64_t prow = ((int64_t)split * p.B * p.Hkv + group) * p.R + row;
      float* po = p.part_o + prow * D;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          f32x4_t w4 = {o[dt][4 * a], o[dt][4 * a + 1], o[dt][4 * a + 2], o[dt][4 * a + 3]};
          *(f32x4_t*)(po + dt * 32 + 8 * a + 4 * h) = w4;
        }
      if (h == 0) {
        p.part_ml[prow * 2] = m * p.c;  // -inf if the split saw no visible key
        p.part_ml[prow * 2 + 1] = lt;
      }
    }
  }
}

// Combine the per-split partials of a row: one workgroup of D/4 threads... one thread per 4 d.
template <int D, bool F16>
__global__ __launch_bounds__(256) void sdpa_prefill_merge_kernel(const PrefillParams p) {
  constexpr int TPR = D / 4;              // threads per row
  constexpr int ROWS = 256 / TPR;         // rows per workgroup
  const int64_t total_rows = (int64_t)p.B * p.Hkv * p.R;
  const int64_t grow = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR;
  if (grow >= total_rows) return;
  const int dq = threadIdx.x % TPR;
  const int group = (int)(grow / p.R);
  const int row = (int)(grow % p.R);
  const int b = group / p.Hkv, kvh = group % p.Hkv;
  const int qi = row / p.G, g = row % p.G;
  float M = -INFINITY;
  for (int s = 0; s < p.num_splits; ++s) M = fmaxf(M, p.part_ml[((int64_t)s * total_rows + grow) * 2]);
  const float Mu = (M == -INFINITY) ? 0.0f : M;
  float L = 0.0f;
  f32x4_t acc = {0, 0, 0, 0};
  for (int s = 0; s < p.num_splits; ++s) {
    const int64_t pr = (int64_t)s * total_rows + grow;
    const float w = fast_exp2(p.part_ml[pr * 2] - Mu);
    L += p.part_ml[pr * 2 + 1] * w;
    const f32x4_t x = *(const f32x4_t*)(p.part_o + pr * D + dq * 4);
    acc += x * w;
  }
  const float inv = L > 0.0f ? 1.0f / L : 0.0f;
  uint16_t* op = p.o + b * p.o_sb + (int64_t)(kvh * p.G + g) * p.o_sh + (int64_t)qi * p.o_st + dq * 4;
  u32x2_t w2;
  w2[0] = pack_pair<F16>(acc[0] * inv, acc[1] * inv);
  w2[1] = pack_pair<F16>(acc[2] * inv, acc[3] * inv);
  *(u32x2_t*)op = w2;
  if (p.lse && dq == 0) p.lse[((int64_t)b * p.q_len + qi) * p.Hq + kvh * p.G + g] = Mu + fast_log2(L);
}

int pick_splits(const kvx_sdpa_args& a, int m_blocks, int num_tiles) {
  if (a.num_splits > 0) return min(a.num_splits, num_tiles);
  // Aim for one resident round of workgroups (2 per compute unit, 1 with the uint8 cache): more
  // splits only add partials to write, merge and re-read. At least 8 key tiles per split.
  const int64_t base = (int64_t)a.B * a.Hkv * m_blocks;
  const int target = ((kv_is_plain(a.kv_dtype) && a.D <= 128) ? 2 : 1) * num_cus();
  int s = (int)((target + base - 1) / base);
  s = max(1, min(s, num_tiles / 8));
  return max(1, min(s, 64));
}

void fill_params(PrefillParams& p, const kvx_sdpa_args& a) {
  p.q = (const uint16_t*)a.q;
  p.k = a.k;
  p.v = a.v;
  p.k_scale = a.k_scale;
  p.k_zp = a.k_zp;
  p.v_scale = a.v_scale;
  p.v_zp = a.v_zp;
  p.tp = a.token_positions;
  p.o = (uint16_t*)a.o;
  p.lse = a.lse;
  p.B = a.B;
  p.Hq = a.Hq;
  p.Hkv = a.Hkv;
  p.G = a.Hq / a.Hkv;
  p.q_len = a.q_len;
  p.kv_len = a.kv_len;
  p.R = a.q_len * p.G;
  p.input_pos = a.input_pos;
  p.num_tiles = (a.kv_len + BN - 1) / BN;
  const int bm = 32 * nwaves(a.kv_dtype, a.D);
  p.m_blocks = (p.R + bm - 1) / bm;
  p.num_splits = pick_splits(a, p.m_blocks, p.num_tiles);
  p.tiles_per_split = (p.num_tiles + p.num_splits - 1) / p.num_splits;
  p.num_splits = (p.num_tiles + p.tiles_per_split - 1) / p.tiles_per_split;
  p.c = a.sm_scale * kLog2e;
  p.q_sb = a.q_stride_b; p.q_sh = a.q_stride_h; p.q_st = a.q_stride_t;
  p.k_sb = a.k_stride_b; p.k_sh = a.k_stride_h; p.k_st = a.k_stride_t;
  p.v_sb = a.v_stride_b; p.v_sh = a.v_stride_h; p.v_st = a.v_stride_t;
  p.o_sb = a.o_stride_b; p.o_sh = a.o_stride_h; p.o_st = a.o_stride_t;
  p.qs_sb = a.qs_stride_b; p.qs_sh = a.qs_stride_h;
  p.tp_sb = a.tp_stride_b; p.tp_sh = a.tp_stride_h;
  p.part_o = nullptr;
  p.part_ml = nullptr;
}

size_t partial_bytes(const PrefillParams& p, int D) {
  if (p.num_splits <= 1) return 0;
  const size_t rows = (size_t)p.num_splits * p.B * p.Hkv * p.R;
  return rows * (size_t)D * 4 + rows * 2 * 4;
}

template <int D, int KV>
int launch_t(PrefillParams& p, hipStream_t st) {
  dim3 grid(p.B * p.Hkv, p.m_blocks, p.num_splits);
  hipLaunchKernelGGL((sdpa_prefill_kernel<D, KV>), grid, dim3(64 * nwaves(KV, D)), 0, st, p);
  KVX_HIP(hipGetLastError());
  if (p.num_splits > 1) {
    constexpr int ROWS = 256 / (D / 4);
    const int64_t total_rows = (int64_t)p.B * p.Hkv * p.R;
    hipLaunchKernelGGL((sdpa_prefill_merge_kernel<D, kv_elem_f16(KV)>), dim3((unsigned)((total_rows + ROWS - 1) / ROWS)), dim3(256), 0, st, p);
    KVX_HIP(hipGetLastError());
  }
  return KVX_OK;
}

}  // namespace

size_t sdpa_prefill_workspace(const kvx_sdpa_args& a) {
  PrefillParams p;
  fill_params(p, a);
  // the score-sum pass that may follow on the same stream reuses the workspace for its partial sums
  const size_t own = partial_bytes(p, a.D), after = score_sum_workspace(a);
  return own > after ? own : after;
}

int launch_sdpa_prefill(const kvx_sdpa_args& a, hipStream_t st) {
  PrefillParams p;
  fill_params(p, a);
  const size_t need = partial_bytes(p, a.D);
  if (need) {
    KVX_REQUIRE(a.workspace && a.workspace_bytes >= need, KVX_ERR_WORKSPACE,
                "kvx_sdpa_prefill: workspace of %zu bytes needed, %zu given", need, a.workspace_bytes);
    const size_t rows = (size_t)p.num_splits * p.B * p.Hkv * p.R;
    p.part_o = (float*)a.workspace;
    p.part_ml = p.part_o + rows * (size_t)a.D;
  }
#define KVX_PREFILL_CASE(KV) \
  case KV: return a.D == 256 ? launch_t<256, KV>(p, st) : a.D == 128 ? launch_t<128, KV>(p, st) : launch_t<64, KV>(p, st);
  if (a.D == 256 || a.D == 128 || a.D == 64) {
    switch (a.kv_dtype) {
      KVX_PREFILL_CASE(KVX_KV_BF16)
      KVX_PREFILL_CASE(KVX_KV_F16)
      KVX_PREFILL_CASE(KVX_KV_U8)
      KVX_PREFILL_CASE(KVX_KV_U4)
      KVX_PREFILL_CASE(KVX_KV_U8_F16)
      KVX_PREFILL_CASE(KVX_KV_U4_F16)
    }
  }
#undef KVX_PREFILL_CASE
  return set_error(KVX_ERR_UNSUPPORTED, "kvx_sdpa_prefill: head size %d not in {64, 128, 256}", a.D);
}

}  // namespace kvx
