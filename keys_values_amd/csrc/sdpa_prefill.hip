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
#include <cstdlib>
#include <cstring>
#include <type_traits>
#include <utility>

#include "kvx_common.h"

namespace kvx {
namespace {

constexpr float kSlackLog2 = 8.0f;  // see the running-maximum update in the kernel

// Wavefronts per workgroup, 32 rows each. The uint8 cache takes 8: a tile is dequantised once per
// workgroup, so twice the rows halve that vector work per row (-13 % kernel time); for bf16 tiles the
// two sizes run alike and the smaller one leaves more workgroups for short chunks.
constexpr int nwaves(int kv) { return kv_is_plain(kv) ? 4 : 8; }  // kv: enum kvx_kv_dtype
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
  int32_t tp[4][BN];  // token positions of the K tiles: the buffer of the tile, or a ring of four (64-row kernel)
};

typedef short s16x4_t __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i (a = i % 4, r = i / 4) supplies the
// address of 4 consecutive bf16 of "row r, columns 4a..4a+3"; it receives column i of rows 0..3.
typedef char __attribute__((address_space(3))) * lds_ptr_t;
__device__ __forceinline__ u32x2_t lds_read_tr16(lds_ptr_t p) {
  const s16x4_t t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)(p));
  return __builtin_bit_cast(u32x2_t, t);
}

// 16 bytes per lane straight from global memory into LDS (global_load_lds_dwordx4): lane l lands at
// lds_addr + 16 l, lds_addr uniform over the wavefront. Written as inline assembly so that the
// compiler does not serialise later LDS reads of OTHER buffers behind the transfer; the kernel
// waits for its transfers itself (s_waitcnt vmcnt(0)) before the barrier that publishes a tile.
__device__ __forceinline__ void dma16(const char* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(base)
               : "memory", "m0");
}
// the same with the LDS address formed as lds_base + IMM in M0 by the one scalar instruction the
// transfer needs anyway
template <uint32_t IMM>
__device__ __forceinline__ void dma16_at(const char* base, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_base), "v"(voff), "s"(base), "n"(IMM)
               : "memory", "m0", "scc");
}
// same for 4 bytes per lane (global_load_lds_dword): lane l lands at lds_addr + 4 l
__device__ __forceinline__ void dma4(const char* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(base)
               : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_addr_of(const void* p) {
  return (uint32_t)(uintptr_t)((const __attribute__((address_space(3))) char*)p);
}

// 8 codes (two dwords) -> 8 bf16 (four dwords)
__device__ __forceinline__ u32x4_t dequant8(uint32_t c0, uint32_t c1, int32_t zp, float scale) { return dequant_words(c0, c1, zp, scale); }

// Tile loader. A wavefront instruction covers RPW = 64 / CPR whole rows; wavefront w of the
// workgroup takes row groups w, w + 4, ... of the 64-row tile (NI groups each for K and for V).
// bf16 cache: DMA into LDS. uint8 cache: codes and row state go through registers (prefetched one
// tile ahead like the DMA), are dequantised to bf16 and written to the same LDS layout.
template <int D, int KV>
struct Loader {
  static constexpr bool U8 = !kv_is_plain(KV);  // codes through registers (8-bit or 4-bit store)
  static constexpr bool U4 = KV == KVX_KV_U4;
  static constexpr int CPR = D / 8;
  static constexpr int RPW = 64 / CPR;        // rows per wavefront instruction: 4 (D=128), 8 (D=64)
  static constexpr int NWAVES = nwaves(KV);
  static constexpr int NTHREADS = 64 * NWAVES;
  static constexpr int NI = BN / RPW / NWAVES;     // instructions per wavefront per operand: 4 / 2
  static constexpr int ESZ = U8 ? 1 : 2;
  const char* kbase;
  const char* vbase;
  const float* ks;
  const int32_t* kz;
  const float* vs;
  const int32_t* vz;
  const int32_t* tp;
  uint32_t koff, voff;          // byte offset of this lane's chunk of row group 0 inside a tile (source side swizzled)
  int64_t k_tile_bytes, v_tile_bytes, k_st, v_st;
  int64_t k_step, v_step;       // bytes between this wavefront's consecutive row groups (NWAVES RPW rows)
  int wave, lane, kv_len, rl;
  int cgk[NI], cgv[NI];         // the source chunk that belongs at this lane's LDS position, per row group
  int shk, shv;                 // 4-bit store: nibble of this lane's K / V chunk (4 = high)
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
    // row groups of one wavefront are NWAVES RPW rows apart: a multiple of 16 (the XOR keys and with them the
    // source chunks are then the same for all of them) except for D = 256 with four wavefronts (8 rows apart)
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int r = row_of(i);
      cgk[i] = (lane % CPR) ^ swz_k<CPR>(r);  // the chunk that belongs at LDS position lane % CPR of row r
      cgv[i] = (lane % CPR) ^ swz_v<CPR>(r);
    }
    const int r0 = row_of(0);
    koff = (uint32_t)(r0 * p.k_st * ESZ + chunk_off(cgk[0]));
    voff = (uint32_t)(r0 * p.v_st * ESZ + chunk_off(cgv[0]));
    shk = u4_shift<D>(cgk[0]);  // quantised stores: D <= 128, all row groups share their chunk
    shv = u4_shift<D>(cgv[0]);
    k_step = (int64_t)NWAVES * RPW * p.k_st * ESZ;
    v_step = (int64_t)NWAVES * RPW * p.v_st * ESZ;
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

  // tpb: where the tile's token positions go (default: the tile's own buffer index)
  template <bool IS_K>
  __device__ __forceinline__ void issue_one(Smem<D>& sm, int tile, int buf, int tid, int tpb = -1) {
    const int key0 = tile * BN;
    if (tpb < 0) tpb = buf;
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
    const int64_t step = IS_K ? k_step : v_step;
    const uint32_t off0 = IS_K ? koff : voff;
    const char* tb = base + tile * (IS_K ? k_tile_bytes : v_tile_bytes);
    if (key0 + BN <= kv_len) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        if constexpr (!U8) {
          const uint32_t dst = (IS_K ? lds_k : lds_v) + (uint32_t)((buf * BN + (NWAVES * i + wave) * RPW) * CPR * 16);
          dma16(tb, IS_K ? koffs[i] : voffs[i], dst);
        } else {
          const int key = key0 + row_of(i);
          const u32x2_t c = *(const u32x2_t*)(tb + i * step + off0);
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
  __device__ __forceinline__ void land(Smem<D>& sm, int tile, int buf, int tid, int tpb = -1) {
    if (tpb < 0) tpb = buf;
    if constexpr (U8) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int r = row_of(i);
        u32x2_t c = IS_K ? kc[i] : vc[i];
        if constexpr (U4) c = u4_codes(c, IS_K ? shk : shv);
        if (IS_K) sm.k[buf][r][lane % CPR] = dequant8(c[0], c[1], kzr[i], ksr[i]);
        else sm.v[buf][r][lane % CPR] = dequant8(c[0], c[1], vzr[i], vsr[i]);
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
__global__ __launch_bounds__(64 * nwaves(KV), (kv_is_plain(KV) && D <= 128) ? 2 : 1) void sdpa_prefill_kernel(const PrefillParams p) {
  constexpr bool F16 = KV == KVX_KV_F16;  // element type of q, k, v, o
  constexpr int BM = 32 * nwaves(KV);  // rows per workgroup
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

// ---- 64 rows per wavefront -----------------------------------------------------------------------------
//
// The same product for long chunks of plain 16-bit rows with D = 128, arranged so that every K / V fragment
// read from LDS feeds two matrix instructions and every tile that travels to LDS serves 256 rows: four
// wavefronts of 64 rows (two row blocks of 32), one wavefront per SIMD. A wavefront then holds O (128
// registers) and its Q fragments (64) in the accumulation registers, where only the matrix instructions
// touch them, and S / P in the vector registers. With nothing else resident on the SIMD the overlap of the
// matrix core and the vector ALU has to come from this wavefront's own instruction stream: a step is 32
// keys; while the vector ALU turns S(s) into P(s), the matrix core multiplies K(s+1) Q^T into the other
// S buffer and adds V(s-1) P(s-1) to O. Neither depends on the vector work of the same step, so the two
// streams are interleaved instruction by instruction. The matrix instructions are inline assembly (the
// compiler would otherwise keep every accumulator, S included, in the accumulation registers and copy
// S out and P in around each step); the results they leave in vector registers are first read a whole
// step later, far beyond the wait states such a read needs.

template <bool F16>
__device__ __forceinline__ void mfma_s_first(f32x16_t& s, const u32x4_t& k, const u32x4_t& q) {
  if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(s) : "v"(k), "a"(q));
  else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(s) : "v"(k), "a"(q));
}
template <bool F16>
__device__ __forceinline__ void mfma_s(f32x16_t& s, const u32x4_t& k, const u32x4_t& q) {
  if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(s) : "v"(k), "a"(q));
  else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(s) : "v"(k), "a"(q));
}
// O lives in fixed accumulation registers a[0:127], block (dt, rb) in a[16 (2 dt + rb) .. +15]: every statement that
// touches it is inline assembly naming those registers, so the compiler has nothing to copy, spill or reorder.
template <bool F16, int IDX>
__device__ __forceinline__ void mfma_o(f32x16_t& o, const u32x4_t& v, const u32x4_t& pf) {
  if constexpr (IDX == 0) {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+{a[0:15]}"(o) : "v"(v), "v"(pf));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+{a[0:15]}"(o) : "v"(v), "v"(pf));
  }
  else if constexpr (IDX == 1) {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+{a[16:31]}"(o) : "v"(v), "v"(pf));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+{a[16:31]}"(o) : "v"(v), "v"(pf));
  }
  else if constexpr (IDX == 2) {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+{a[32:47]}"(o) : "v"(v), "v"(pf));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+{a[32:47]}"(o) : "v"(v), "v"(pf));
  }
  else if constexpr (IDX == 3) {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+{a[48:63]}"(o) : "v"(v), "v"(pf));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+{a[48:63]}"(o) : "v"(v), "v"(pf));
  }
  else if constexpr (IDX == 4) {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+{a[64:79]}"(o) : "v"(v), "v"(pf));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+{a[64:79]}"(o) : "v"(v), "v"(pf));
  }
  else if constexpr (IDX == 5) {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+{a[80:95]}"(o) : "v"(v), "v"(pf));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+{a[80:95]}"(o) : "v"(v), "v"(pf));
  }
  else if constexpr (IDX == 6) {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+{a[96:111]}"(o) : "v"(v), "v"(pf));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+{a[96:111]}"(o) : "v"(v), "v"(pf));
  }
  else if constexpr (IDX == 7) {
    if constexpr (F16) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+{a[112:127]}"(o) : "v"(v), "v"(pf));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+{a[112:127]}"(o) : "v"(v), "v"(pf));
  }
}
// block IDX *= alpha (per lane: a lane holds one row), through two vector registers
template <int IDX>
__device__ __forceinline__ void scale_o(f32x16_t& o, float alpha) {
  float t0, t1;
  if constexpr (IDX == 0)
    asm volatile("v_accvgpr_read_b32 %1, a0\n\tv_accvgpr_read_b32 %2, a1\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a0, %1\n\tv_accvgpr_write_b32 a1, %2\n\t"
                 "v_accvgpr_read_b32 %1, a2\n\tv_accvgpr_read_b32 %2, a3\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a2, %1\n\tv_accvgpr_write_b32 a3, %2\n\t"
                 "v_accvgpr_read_b32 %1, a4\n\tv_accvgpr_read_b32 %2, a5\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a4, %1\n\tv_accvgpr_write_b32 a5, %2\n\t"
                 "v_accvgpr_read_b32 %1, a6\n\tv_accvgpr_read_b32 %2, a7\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a6, %1\n\tv_accvgpr_write_b32 a7, %2\n\t"
                 "v_accvgpr_read_b32 %1, a8\n\tv_accvgpr_read_b32 %2, a9\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a8, %1\n\tv_accvgpr_write_b32 a9, %2\n\t"
                 "v_accvgpr_read_b32 %1, a10\n\tv_accvgpr_read_b32 %2, a11\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a10, %1\n\tv_accvgpr_write_b32 a11, %2\n\t"
                 "v_accvgpr_read_b32 %1, a12\n\tv_accvgpr_read_b32 %2, a13\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a12, %1\n\tv_accvgpr_write_b32 a13, %2\n\t"
                 "v_accvgpr_read_b32 %1, a14\n\tv_accvgpr_read_b32 %2, a15\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a14, %1\n\tv_accvgpr_write_b32 a15, %2\n\t"
                 "s_nop 1" : "+{a[0:15]}"(o), "=&v"(t0), "=&v"(t1) : "v"(alpha));
  else if constexpr (IDX == 1)
    asm volatile("v_accvgpr_read_b32 %1, a16\n\tv_accvgpr_read_b32 %2, a17\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a16, %1\n\tv_accvgpr_write_b32 a17, %2\n\t"
                 "v_accvgpr_read_b32 %1, a18\n\tv_accvgpr_read_b32 %2, a19\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a18, %1\n\tv_accvgpr_write_b32 a19, %2\n\t"
                 "v_accvgpr_read_b32 %1, a20\n\tv_accvgpr_read_b32 %2, a21\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a20, %1\n\tv_accvgpr_write_b32 a21, %2\n\t"
                 "v_accvgpr_read_b32 %1, a22\n\tv_accvgpr_read_b32 %2, a23\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a22, %1\n\tv_accvgpr_write_b32 a23, %2\n\t"
                 "v_accvgpr_read_b32 %1, a24\n\tv_accvgpr_read_b32 %2, a25\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a24, %1\n\tv_accvgpr_write_b32 a25, %2\n\t"
                 "v_accvgpr_read_b32 %1, a26\n\tv_accvgpr_read_b32 %2, a27\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a26, %1\n\tv_accvgpr_write_b32 a27, %2\n\t"
                 "v_accvgpr_read_b32 %1, a28\n\tv_accvgpr_read_b32 %2, a29\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a28, %1\n\tv_accvgpr_write_b32 a29, %2\n\t"
                 "v_accvgpr_read_b32 %1, a30\n\tv_accvgpr_read_b32 %2, a31\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a30, %1\n\tv_accvgpr_write_b32 a31, %2\n\t"
                 "s_nop 1" : "+{a[16:31]}"(o), "=&v"(t0), "=&v"(t1) : "v"(alpha));
  else if constexpr (IDX == 2)
    asm volatile("v_accvgpr_read_b32 %1, a32\n\tv_accvgpr_read_b32 %2, a33\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a32, %1\n\tv_accvgpr_write_b32 a33, %2\n\t"
                 "v_accvgpr_read_b32 %1, a34\n\tv_accvgpr_read_b32 %2, a35\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a34, %1\n\tv_accvgpr_write_b32 a35, %2\n\t"
                 "v_accvgpr_read_b32 %1, a36\n\tv_accvgpr_read_b32 %2, a37\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a36, %1\n\tv_accvgpr_write_b32 a37, %2\n\t"
                 "v_accvgpr_read_b32 %1, a38\n\tv_accvgpr_read_b32 %2, a39\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a38, %1\n\tv_accvgpr_write_b32 a39, %2\n\t"
                 "v_accvgpr_read_b32 %1, a40\n\tv_accvgpr_read_b32 %2, a41\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a40, %1\n\tv_accvgpr_write_b32 a41, %2\n\t"
                 "v_accvgpr_read_b32 %1, a42\n\tv_accvgpr_read_b32 %2, a43\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a42, %1\n\tv_accvgpr_write_b32 a43, %2\n\t"
                 "v_accvgpr_read_b32 %1, a44\n\tv_accvgpr_read_b32 %2, a45\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a44, %1\n\tv_accvgpr_write_b32 a45, %2\n\t"
                 "v_accvgpr_read_b32 %1, a46\n\tv_accvgpr_read_b32 %2, a47\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a46, %1\n\tv_accvgpr_write_b32 a47, %2\n\t"
                 "s_nop 1" : "+{a[32:47]}"(o), "=&v"(t0), "=&v"(t1) : "v"(alpha));
  else if constexpr (IDX == 3)
    asm volatile("v_accvgpr_read_b32 %1, a48\n\tv_accvgpr_read_b32 %2, a49\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a48, %1\n\tv_accvgpr_write_b32 a49, %2\n\t"
                 "v_accvgpr_read_b32 %1, a50\n\tv_accvgpr_read_b32 %2, a51\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a50, %1\n\tv_accvgpr_write_b32 a51, %2\n\t"
                 "v_accvgpr_read_b32 %1, a52\n\tv_accvgpr_read_b32 %2, a53\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a52, %1\n\tv_accvgpr_write_b32 a53, %2\n\t"
                 "v_accvgpr_read_b32 %1, a54\n\tv_accvgpr_read_b32 %2, a55\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a54, %1\n\tv_accvgpr_write_b32 a55, %2\n\t"
                 "v_accvgpr_read_b32 %1, a56\n\tv_accvgpr_read_b32 %2, a57\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a56, %1\n\tv_accvgpr_write_b32 a57, %2\n\t"
                 "v_accvgpr_read_b32 %1, a58\n\tv_accvgpr_read_b32 %2, a59\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a58, %1\n\tv_accvgpr_write_b32 a59, %2\n\t"
                 "v_accvgpr_read_b32 %1, a60\n\tv_accvgpr_read_b32 %2, a61\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a60, %1\n\tv_accvgpr_write_b32 a61, %2\n\t"
                 "v_accvgpr_read_b32 %1, a62\n\tv_accvgpr_read_b32 %2, a63\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a62, %1\n\tv_accvgpr_write_b32 a63, %2\n\t"
                 "s_nop 1" : "+{a[48:63]}"(o), "=&v"(t0), "=&v"(t1) : "v"(alpha));
  else if constexpr (IDX == 4)
    asm volatile("v_accvgpr_read_b32 %1, a64\n\tv_accvgpr_read_b32 %2, a65\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a64, %1\n\tv_accvgpr_write_b32 a65, %2\n\t"
                 "v_accvgpr_read_b32 %1, a66\n\tv_accvgpr_read_b32 %2, a67\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a66, %1\n\tv_accvgpr_write_b32 a67, %2\n\t"
                 "v_accvgpr_read_b32 %1, a68\n\tv_accvgpr_read_b32 %2, a69\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a68, %1\n\tv_accvgpr_write_b32 a69, %2\n\t"
                 "v_accvgpr_read_b32 %1, a70\n\tv_accvgpr_read_b32 %2, a71\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a70, %1\n\tv_accvgpr_write_b32 a71, %2\n\t"
                 "v_accvgpr_read_b32 %1, a72\n\tv_accvgpr_read_b32 %2, a73\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a72, %1\n\tv_accvgpr_write_b32 a73, %2\n\t"
                 "v_accvgpr_read_b32 %1, a74\n\tv_accvgpr_read_b32 %2, a75\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a74, %1\n\tv_accvgpr_write_b32 a75, %2\n\t"
                 "v_accvgpr_read_b32 %1, a76\n\tv_accvgpr_read_b32 %2, a77\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a76, %1\n\tv_accvgpr_write_b32 a77, %2\n\t"
                 "v_accvgpr_read_b32 %1, a78\n\tv_accvgpr_read_b32 %2, a79\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a78, %1\n\tv_accvgpr_write_b32 a79, %2\n\t"
                 "s_nop 1" : "+{a[64:79]}"(o), "=&v"(t0), "=&v"(t1) : "v"(alpha));
  else if constexpr (IDX == 5)
    asm volatile("v_accvgpr_read_b32 %1, a80\n\tv_accvgpr_read_b32 %2, a81\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a80, %1\n\tv_accvgpr_write_b32 a81, %2\n\t"
                 "v_accvgpr_read_b32 %1, a82\n\tv_accvgpr_read_b32 %2, a83\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a82, %1\n\tv_accvgpr_write_b32 a83, %2\n\t"
                 "v_accvgpr_read_b32 %1, a84\n\tv_accvgpr_read_b32 %2, a85\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a84, %1\n\tv_accvgpr_write_b32 a85, %2\n\t"
                 "v_accvgpr_read_b32 %1, a86\n\tv_accvgpr_read_b32 %2, a87\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a86, %1\n\tv_accvgpr_write_b32 a87, %2\n\t"
                 "v_accvgpr_read_b32 %1, a88\n\tv_accvgpr_read_b32 %2, a89\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a88, %1\n\tv_accvgpr_write_b32 a89, %2\n\t"
                 "v_accvgpr_read_b32 %1, a90\n\tv_accvgpr_read_b32 %2, a91\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a90, %1\n\tv_accvgpr_write_b32 a91, %2\n\t"
                 "v_accvgpr_read_b32 %1, a92\n\tv_accvgpr_read_b32 %2, a93\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a92, %1\n\tv_accvgpr_write_b32 a93, %2\n\t"
                 "v_accvgpr_read_b32 %1, a94\n\tv_accvgpr_read_b32 %2, a95\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a94, %1\n\tv_accvgpr_write_b32 a95, %2\n\t"
                 "s_nop 1" : "+{a[80:95]}"(o), "=&v"(t0), "=&v"(t1) : "v"(alpha));
  else if constexpr (IDX == 6)
    asm volatile("v_accvgpr_read_b32 %1, a96\n\tv_accvgpr_read_b32 %2, a97\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a96, %1\n\tv_accvgpr_write_b32 a97, %2\n\t"
                 "v_accvgpr_read_b32 %1, a98\n\tv_accvgpr_read_b32 %2, a99\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a98, %1\n\tv_accvgpr_write_b32 a99, %2\n\t"
                 "v_accvgpr_read_b32 %1, a100\n\tv_accvgpr_read_b32 %2, a101\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a100, %1\n\tv_accvgpr_write_b32 a101, %2\n\t"
                 "v_accvgpr_read_b32 %1, a102\n\tv_accvgpr_read_b32 %2, a103\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a102, %1\n\tv_accvgpr_write_b32 a103, %2\n\t"
                 "v_accvgpr_read_b32 %1, a104\n\tv_accvgpr_read_b32 %2, a105\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a104, %1\n\tv_accvgpr_write_b32 a105, %2\n\t"
                 "v_accvgpr_read_b32 %1, a106\n\tv_accvgpr_read_b32 %2, a107\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a106, %1\n\tv_accvgpr_write_b32 a107, %2\n\t"
                 "v_accvgpr_read_b32 %1, a108\n\tv_accvgpr_read_b32 %2, a109\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a108, %1\n\tv_accvgpr_write_b32 a109, %2\n\t"
                 "v_accvgpr_read_b32 %1, a110\n\tv_accvgpr_read_b32 %2, a111\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a110, %1\n\tv_accvgpr_write_b32 a111, %2\n\t"
                 "s_nop 1" : "+{a[96:111]}"(o), "=&v"(t0), "=&v"(t1) : "v"(alpha));
  else if constexpr (IDX == 7)
    asm volatile("v_accvgpr_read_b32 %1, a112\n\tv_accvgpr_read_b32 %2, a113\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a112, %1\n\tv_accvgpr_write_b32 a113, %2\n\t"
                 "v_accvgpr_read_b32 %1, a114\n\tv_accvgpr_read_b32 %2, a115\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a114, %1\n\tv_accvgpr_write_b32 a115, %2\n\t"
                 "v_accvgpr_read_b32 %1, a116\n\tv_accvgpr_read_b32 %2, a117\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a116, %1\n\tv_accvgpr_write_b32 a117, %2\n\t"
                 "v_accvgpr_read_b32 %1, a118\n\tv_accvgpr_read_b32 %2, a119\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a118, %1\n\tv_accvgpr_write_b32 a119, %2\n\t"
                 "v_accvgpr_read_b32 %1, a120\n\tv_accvgpr_read_b32 %2, a121\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a120, %1\n\tv_accvgpr_write_b32 a121, %2\n\t"
                 "v_accvgpr_read_b32 %1, a122\n\tv_accvgpr_read_b32 %2, a123\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a122, %1\n\tv_accvgpr_write_b32 a123, %2\n\t"
                 "v_accvgpr_read_b32 %1, a124\n\tv_accvgpr_read_b32 %2, a125\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a124, %1\n\tv_accvgpr_write_b32 a125, %2\n\t"
                 "v_accvgpr_read_b32 %1, a126\n\tv_accvgpr_read_b32 %2, a127\n\tv_mul_f32 %1, %1, %3\n\tv_mul_f32 %2, %2, %3\n\tv_accvgpr_write_b32 a126, %1\n\tv_accvgpr_write_b32 a127, %2\n\t"
                 "s_nop 1" : "+{a[112:127]}"(o), "=&v"(t0), "=&v"(t1) : "v"(alpha));
}
// block IDX = 0
template <int IDX>
__device__ __forceinline__ void zero_o(f32x16_t& o) {
  if constexpr (IDX == 0)
    asm volatile("v_accvgpr_write_b32 a0, 0\n\t"
                 "v_accvgpr_write_b32 a1, 0\n\t"
                 "v_accvgpr_write_b32 a2, 0\n\t"
                 "v_accvgpr_write_b32 a3, 0\n\t"
                 "v_accvgpr_write_b32 a4, 0\n\t"
                 "v_accvgpr_write_b32 a5, 0\n\t"
                 "v_accvgpr_write_b32 a6, 0\n\t"
                 "v_accvgpr_write_b32 a7, 0\n\t"
                 "v_accvgpr_write_b32 a8, 0\n\t"
                 "v_accvgpr_write_b32 a9, 0\n\t"
                 "v_accvgpr_write_b32 a10, 0\n\t"
                 "v_accvgpr_write_b32 a11, 0\n\t"
                 "v_accvgpr_write_b32 a12, 0\n\t"
                 "v_accvgpr_write_b32 a13, 0\n\t"
                 "v_accvgpr_write_b32 a14, 0\n\t"
                 "v_accvgpr_write_b32 a15, 0\n\t"
                 "s_nop 1" : "={a[0:15]}"(o));
  else if constexpr (IDX == 1)
    asm volatile("v_accvgpr_write_b32 a16, 0\n\t"
                 "v_accvgpr_write_b32 a17, 0\n\t"
                 "v_accvgpr_write_b32 a18, 0\n\t"
                 "v_accvgpr_write_b32 a19, 0\n\t"
                 "v_accvgpr_write_b32 a20, 0\n\t"
                 "v_accvgpr_write_b32 a21, 0\n\t"
                 "v_accvgpr_write_b32 a22, 0\n\t"
                 "v_accvgpr_write_b32 a23, 0\n\t"
                 "v_accvgpr_write_b32 a24, 0\n\t"
                 "v_accvgpr_write_b32 a25, 0\n\t"
                 "v_accvgpr_write_b32 a26, 0\n\t"
                 "v_accvgpr_write_b32 a27, 0\n\t"
                 "v_accvgpr_write_b32 a28, 0\n\t"
                 "v_accvgpr_write_b32 a29, 0\n\t"
                 "v_accvgpr_write_b32 a30, 0\n\t"
                 "v_accvgpr_write_b32 a31, 0\n\t"
                 "s_nop 1" : "={a[16:31]}"(o));
  else if constexpr (IDX == 2)
    asm volatile("v_accvgpr_write_b32 a32, 0\n\t"
                 "v_accvgpr_write_b32 a33, 0\n\t"
                 "v_accvgpr_write_b32 a34, 0\n\t"
                 "v_accvgpr_write_b32 a35, 0\n\t"
                 "v_accvgpr_write_b32 a36, 0\n\t"
                 "v_accvgpr_write_b32 a37, 0\n\t"
                 "v_accvgpr_write_b32 a38, 0\n\t"
                 "v_accvgpr_write_b32 a39, 0\n\t"
                 "v_accvgpr_write_b32 a40, 0\n\t"
                 "v_accvgpr_write_b32 a41, 0\n\t"
                 "v_accvgpr_write_b32 a42, 0\n\t"
                 "v_accvgpr_write_b32 a43, 0\n\t"
                 "v_accvgpr_write_b32 a44, 0\n\t"
                 "v_accvgpr_write_b32 a45, 0\n\t"
                 "v_accvgpr_write_b32 a46, 0\n\t"
                 "v_accvgpr_write_b32 a47, 0\n\t"
                 "s_nop 1" : "={a[32:47]}"(o));
  else if constexpr (IDX == 3)
    asm volatile("v_accvgpr_write_b32 a48, 0\n\t"
                 "v_accvgpr_write_b32 a49, 0\n\t"
                 "v_accvgpr_write_b32 a50, 0\n\t"
                 "v_accvgpr_write_b32 a51, 0\n\t"
                 "v_accvgpr_write_b32 a52, 0\n\t"
                 "v_accvgpr_write_b32 a53, 0\n\t"
                 "v_accvgpr_write_b32 a54, 0\n\t"
                 "v_accvgpr_write_b32 a55, 0\n\t"
                 "v_accvgpr_write_b32 a56, 0\n\t"
                 "v_accvgpr_write_b32 a57, 0\n\t"
                 "v_accvgpr_write_b32 a58, 0\n\t"
                 "v_accvgpr_write_b32 a59, 0\n\t"
                 "v_accvgpr_write_b32 a60, 0\n\t"
                 "v_accvgpr_write_b32 a61, 0\n\t"
                 "v_accvgpr_write_b32 a62, 0\n\t"
                 "v_accvgpr_write_b32 a63, 0\n\t"
                 "s_nop 1" : "={a[48:63]}"(o));
  else if constexpr (IDX == 4)
    asm volatile("v_accvgpr_write_b32 a64, 0\n\t"
                 "v_accvgpr_write_b32 a65, 0\n\t"
                 "v_accvgpr_write_b32 a66, 0\n\t"
                 "v_accvgpr_write_b32 a67, 0\n\t"
                 "v_accvgpr_write_b32 a68, 0\n\t"
                 "v_accvgpr_write_b32 a69, 0\n\t"
                 "v_accvgpr_write_b32 a70, 0\n\t"
                 "v_accvgpr_write_b32 a71, 0\n\t"
                 "v_accvgpr_write_b32 a72, 0\n\t"
                 "v_accvgpr_write_b32 a73, 0\n\t"
                 "v_accvgpr_write_b32 a74, 0\n\t"
                 "v_accvgpr_write_b32 a75, 0\n\t"
                 "v_accvgpr_write_b32 a76, 0\n\t"
                 "v_accvgpr_write_b32 a77, 0\n\t"
                 "v_accvgpr_write_b32 a78, 0\n\t"
                 "v_accvgpr_write_b32 a79, 0\n\t"
                 "s_nop 1" : "={a[64:79]}"(o));
  else if constexpr (IDX == 5)
    asm volatile("v_accvgpr_write_b32 a80, 0\n\t"
                 "v_accvgpr_write_b32 a81, 0\n\t"
                 "v_accvgpr_write_b32 a82, 0\n\t"
                 "v_accvgpr_write_b32 a83, 0\n\t"
                 "v_accvgpr_write_b32 a84, 0\n\t"
                 "v_accvgpr_write_b32 a85, 0\n\t"
                 "v_accvgpr_write_b32 a86, 0\n\t"
                 "v_accvgpr_write_b32 a87, 0\n\t"
                 "v_accvgpr_write_b32 a88, 0\n\t"
                 "v_accvgpr_write_b32 a89, 0\n\t"
                 "v_accvgpr_write_b32 a90, 0\n\t"
                 "v_accvgpr_write_b32 a91, 0\n\t"
                 "v_accvgpr_write_b32 a92, 0\n\t"
                 "v_accvgpr_write_b32 a93, 0\n\t"
                 "v_accvgpr_write_b32 a94, 0\n\t"
                 "v_accvgpr_write_b32 a95, 0\n\t"
                 "s_nop 1" : "={a[80:95]}"(o));
  else if constexpr (IDX == 6)
    asm volatile("v_accvgpr_write_b32 a96, 0\n\t"
                 "v_accvgpr_write_b32 a97, 0\n\t"
                 "v_accvgpr_write_b32 a98, 0\n\t"
                 "v_accvgpr_write_b32 a99, 0\n\t"
                 "v_accvgpr_write_b32 a100, 0\n\t"
                 "v_accvgpr_write_b32 a101, 0\n\t"
                 "v_accvgpr_write_b32 a102, 0\n\t"
                 "v_accvgpr_write_b32 a103, 0\n\t"
                 "v_accvgpr_write_b32 a104, 0\n\t"
                 "v_accvgpr_write_b32 a105, 0\n\t"
                 "v_accvgpr_write_b32 a106, 0\n\t"
                 "v_accvgpr_write_b32 a107, 0\n\t"
                 "v_accvgpr_write_b32 a108, 0\n\t"
                 "v_accvgpr_write_b32 a109, 0\n\t"
                 "v_accvgpr_write_b32 a110, 0\n\t"
                 "v_accvgpr_write_b32 a111, 0\n\t"
                 "s_nop 1" : "={a[96:111]}"(o));
  else if constexpr (IDX == 7)
    asm volatile("v_accvgpr_write_b32 a112, 0\n\t"
                 "v_accvgpr_write_b32 a113, 0\n\t"
                 "v_accvgpr_write_b32 a114, 0\n\t"
                 "v_accvgpr_write_b32 a115, 0\n\t"
                 "v_accvgpr_write_b32 a116, 0\n\t"
                 "v_accvgpr_write_b32 a117, 0\n\t"
                 "v_accvgpr_write_b32 a118, 0\n\t"
                 "v_accvgpr_write_b32 a119, 0\n\t"
                 "v_accvgpr_write_b32 a120, 0\n\t"
                 "v_accvgpr_write_b32 a121, 0\n\t"
                 "v_accvgpr_write_b32 a122, 0\n\t"
                 "v_accvgpr_write_b32 a123, 0\n\t"
                 "v_accvgpr_write_b32 a124, 0\n\t"
                 "v_accvgpr_write_b32 a125, 0\n\t"
                 "v_accvgpr_write_b32 a126, 0\n\t"
                 "v_accvgpr_write_b32 a127, 0\n\t"
                 "s_nop 1" : "={a[112:127]}"(o));
}
// wait states that pass all of O through: whatever reads it afterwards depends on these
__device__ __forceinline__ void settle_o(f32x16_t (&o)[8]) {
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 7"
               : "+{a[0:15]}"(o[0]), "+{a[16:31]}"(o[1]), "+{a[32:47]}"(o[2]), "+{a[48:63]}"(o[3]), "+{a[64:79]}"(o[4]),
                 "+{a[80:95]}"(o[5]), "+{a[96:111]}"(o[6]), "+{a[112:127]}"(o[7]));
}
__device__ __forceinline__ void settle_o(f32x16_t (&o)[4]) {
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 7" : "+{a[0:15]}"(o[0]), "+{a[16:31]}"(o[1]), "+{a[32:47]}"(o[2]), "+{a[48:63]}"(o[3]));
}
// maxima without the canonicalising copies the compiler puts in front of fmaxf (the scores hold no signalling NaN)
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// maximum of a lane's 16 scores and of the other half-wavefront's lane for the same row, as one block (between
// separate statements the compiler would add wait states it cannot know to be unnecessary)
__device__ __forceinline__ float row_max_raw(const f32x16_t& s) {
  float r, t1, t2, t3, t4;
  asm("v_max3_f32 %0, %5, %6, %7\n\t"
      "v_max3_f32 %1, %8, %9, %10\n\t"
      "v_max3_f32 %2, %11, %12, %13\n\t"
      "v_max3_f32 %3, %14, %15, %16\n\t"
      "v_max3_f32 %4, %17, %18, %19\n\t"
      "v_max3_f32 %0, %0, %1, %20\n\t"
      "v_max3_f32 %2, %2, %3, %4\n\t"
      "v_max_f32 %0, %0, %2\n\t"
      "v_mov_b32 %1, %0\n\t"
      "s_nop 1\n\t"
      "v_permlane32_swap_b32 %0, %1\n\t"
      "v_max_f32 %0, %0, %1"
      : "=&v"(r), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4)
      : "v"(s[0]), "v"(s[1]), "v"(s[2]), "v"(s[3]), "v"(s[4]), "v"(s[5]), "v"(s[6]), "v"(s[7]), "v"(s[8]), "v"(s[9]), "v"(s[10]),
        "v"(s[11]), "v"(s[12]), "v"(s[13]), "v"(s[14]), "v"(s[15]));
  return r;
}
__device__ __forceinline__ float max2_raw(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// The compiler takes the result of an inline-assembly matrix instruction for finished when the statement
// ends, and a value for ready for such an instruction as soon as it is written: it places no wait states
// around them. Whatever of its own it puts next to one (copies where control flow joins, arithmetic it
// moved across a barrier) can therefore read a result that is still on its way, or hand over an operand
// too early. These fences keep its code away: wait states that pass O through (everything that reads O
// afterwards depends on them), and empty statements that pin where S and P are complete.
template <class F, int... I>
__device__ __forceinline__ void unroll_seq_impl(F& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, B>), ..., f(integral_constant<int, B + N - 1>)
template <int B, int N, class F>
__device__ __forceinline__ void unroll_seq(F& f) {
  static_assert(B == 0, "sequences start at 0");
  unroll_seq_impl(f, std::make_integer_sequence<int, N>{});
}
__device__ __forceinline__ void pin_s(f32x16_t (&s)[2]) { asm volatile("" : "+v"(s[0]), "+v"(s[1])); }
__device__ __forceinline__ void pin_s(f32x16_t (&s)[1]) { asm volatile("" : "+v"(s[0])); }
__device__ __forceinline__ void pin_p(u32x4_t (&pp)[2][2]) { asm volatile("" : "+v"(pp[0][0]), "+v"(pp[0][1]), "+v"(pp[1][0]), "+v"(pp[1][1])); }
__device__ __forceinline__ void pin_p(u32x4_t (&pp)[1][2]) { asm volatile("" : "+v"(pp[0][0]), "+v"(pp[0][1])); }

constexpr int W64_BM = 256;  // rows per workgroup of the 64-row kernel

// Tile transfers of the 64-row kernel (bf16 / fp16 rows of 128 values, four wavefronts): a wavefront instruction
// moves four whole rows, wavefront w takes rows 4 w .. 4 w + 3 of each 16-row group of the 64-row tile. Rows 16
// apart share their XOR key, so one byte offset per lane serves all four groups of an operand; everything else
// is wavefront-uniform and lives in scalar registers.
struct TileSender {
  static constexpr int CPR = 16;
  const char* kbase;
  const char* vbase;
  const int32_t* tp;
  int64_t k_tile_bytes, v_tile_bytes, k_group_bytes, v_group_bytes, k_row_bytes, v_row_bytes;
  uint32_t koff, voff;      // this lane's chunk in row 4 w + lane / 16 of a tile (source side swizzled)
  uint32_t lds_kw, lds_vw;  // LDS address of row 4 w of buffer 0
  int kv_len, wave;
  // tiles are sent in order: the next K and V tile to send and where they start
  int k_tile, v_tile;
  const char* k_ptr;
  const char* v_ptr;

  __device__ __forceinline__ void init(const PrefillParams& p, Smem<128>& sm, int b, int kvh, int tid, int first_tile) {
    wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    kv_len = p.kv_len;
    kbase = (const char*)p.k + (b * p.k_sb + kvh * p.k_sh) * 2;
    vbase = (const char*)p.v + (b * p.v_sb + kvh * p.v_sh) * 2;
    tp = p.tp ? p.tp + b * p.tp_sb + kvh * p.tp_sh : nullptr;
    k_row_bytes = p.k_st * 2;
    v_row_bytes = p.v_st * 2;
    k_tile_bytes = BN * k_row_bytes;
    v_tile_bytes = BN * v_row_bytes;
    k_group_bytes = 16 * k_row_bytes;
    v_group_bytes = 16 * v_row_bytes;
    const int lane = tid & 63;
    const int r0 = wave * 4 + lane / CPR;
    koff = (uint32_t)(r0 * k_row_bytes) + (uint32_t)(((lane % CPR) ^ swz_k<CPR>(r0)) * 16);
    voff = (uint32_t)(r0 * v_row_bytes) + (uint32_t)(((lane % CPR) ^ swz_v<CPR>(r0)) * 16);
    lds_kw = __builtin_amdgcn_readfirstlane(lds_addr_of(&sm.k[0][0][0])) + (uint32_t)(wave * 4 * CPR * 16);
    lds_vw = __builtin_amdgcn_readfirstlane(lds_addr_of(&sm.v[0][0][0])) + (uint32_t)(wave * 4 * CPR * 16);
    k_tile = v_tile = first_tile;
    k_ptr = kbase + first_tile * k_tile_bytes;
    v_ptr = vbase + first_tile * v_tile_bytes;
  }

  // 16 bytes per lane from base + off to this wavefront's rows of row group I of buffer BUF
  template <bool IS_K, int BUF, int I>
  __device__ __forceinline__ void send_group(const char* base, uint32_t off) {
    dma16_at<(uint32_t)((BUF * BN + 16 * I) * CPR * 16)>(base, off, IS_K ? lds_kw : lds_vw);
  }
  // the next tile of K (with its token positions, into ring slot tps) or V into LDS buffer BUF, if the walk
  // (which ends before tile_end) has one
  template <bool IS_K, int BUF>
  __device__ __forceinline__ void send(Smem<128>& sm, int tid, int tps, int tile_end) {
    const int tile = IS_K ? k_tile : v_tile;
    const char* tb = IS_K ? k_ptr : v_ptr;
    if (IS_K) { ++k_tile; k_ptr += k_tile_bytes; }
    else { ++v_tile; v_ptr += v_tile_bytes; }
    if (tile >= tile_end) return;
    const int key0 = tile * BN;
    if (key0 + BN <= kv_len) {
      const uint32_t off = IS_K ? koff : voff;
      const int64_t gb = IS_K ? k_group_bytes : v_group_bytes;
      send_group<IS_K, BUF, 0>(tb, off);
      send_group<IS_K, BUF, 1>(tb + gb, off);
      send_group<IS_K, BUF, 2>(tb + 2 * gb, off);
      send_group<IS_K, BUF, 3>(tb + 3 * gb, off);
    } else {
      // last, partial tile: rows past the end re-read the last valid row (finite data); their position is
      // INT_MAX, so they are masked for every query and contribute exactly zero
      const int lane = tid & 63;
      const int r0 = wave * 4 + lane / CPR;
      const uint32_t chunk = (uint32_t)(((lane % CPR) ^ (IS_K ? swz_k<CPR>(r0) : swz_v<CPR>(r0))) * 16);
      const int rb = (int)(IS_K ? k_row_bytes : v_row_bytes);
      const int last = kv_len - 1 - key0;
      send_group<IS_K, BUF, 0>(tb, (uint32_t)(min(r0, last) * rb) + chunk);
      send_group<IS_K, BUF, 1>(tb, (uint32_t)(min(r0 + 16, last) * rb) + chunk);
      send_group<IS_K, BUF, 2>(tb, (uint32_t)(min(r0 + 32, last) * rb) + chunk);
      send_group<IS_K, BUF, 3>(tb, (uint32_t)(min(r0 + 48, last) * rb) + chunk);
    }
    if (IS_K && tp && wave == 0) {
      const uint32_t dst = lds_addr_of(&sm.tp[tps][0]);
      dma4((const char*)(tp + key0), (uint32_t)min(tid & 63, kv_len - 1 - key0) * 4, __builtin_amdgcn_readfirstlane(dst));
    }
  }
  // after s_waitcnt vmcnt(0), before the barrier that publishes the K tile: positions of a contiguous cache, and
  // INT_MAX for slots past the end
  // (a tile at or past tile_end is not part of the walk: all its positions are INT_MAX)
  __device__ __forceinline__ void land(Smem<128>& sm, int tile, int tid, int tps, int tile_end) {
    if (tid < BN) {
      const int key = tile * BN + tid;
      const bool hidden = key >= kv_len || tile >= tile_end;
      if (!tp) sm.tp[tps][tid] = hidden ? INT_MAX : key;
      else if (hidden) sm.tp[tps][tid] = INT_MAX;
    }
  }
};

template <int KV, int NRB>
__global__ __launch_bounds__(256, NRB == 1 ? 2 : 1) void sdpa_prefill_slots_kernel(const PrefillParams p) {
  static_assert(NRB == 1 || NRB == 2, "32 or 64 rows per wavefront");
  constexpr int D = 128;
  constexpr bool F16 = KV == KVX_KV_F16;
  constexpr int BM = 128 * NRB;
  constexpr int CPR = D / 8;
  constexpr int KS = D / 16;
  constexpr int DT = D / 32;
  constexpr int NO = DT * NRB;  // blocks of O: block (dt, rb) is o[dt * NRB + rb]
  __shared__ Smem<D> sm;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n = lane & 31;
  const int h = lane >> 5;
  const int group = blockIdx.x;
  const int mblk = blockIdx.y;
  const int split = blockIdx.z;
  const int b = group / p.Hkv;
  const int kvh = group % p.Hkv;

  const int row0w = mblk * BM + wave * 32 * NRB;
  int row[NRB], qi[NRB], g[NRB], qpos[NRB];
  bool row_ok[NRB];
#pragma unroll
  for (int rb = 0; rb < NRB; ++rb) {
    row[rb] = row0w + rb * 32 + n;
    row_ok[rb] = row[rb] < p.R;
    const int rowc = row_ok[rb] ? row[rb] : p.R - 1;
    qi[rb] = rowc / p.G;
    g[rb] = rowc % p.G;
    qpos[rb] = p.input_pos + qi[rb];
  }
  const int qpos_min_w = p.input_pos + min(row0w, p.R - 1) / p.G;

  // Q fragments (B operands): row n of row block rb, d = 16 j + 8 h .. +8. They are loaded straight into
  // accumulation registers (a load may target them) and stay there: a value the compiler first holds in a
  // vector register would be copied over in front of every matrix instruction that reads it. Rows past
  // the end load the last valid row; nothing of theirs is stored.
  u32x4_t qf[NRB][KS];
#pragma unroll
  for (int rb = 0; rb < NRB; ++rb) {
    const uint16_t* qp = p.q + b * p.q_sb + (int64_t)(kvh * p.G + g[rb]) * p.q_sh + (int64_t)qi[rb] * p.q_st + 8 * h;
#pragma unroll
    for (int j = 0; j < KS; ++j) asm volatile("global_load_dwordx4 %0, %1, off" : "=a"(qf[rb][j]) : "v"(qp + 16 * j) : "memory");
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // LDS pointers to this lane's operand fragments in buffer 0 (layout as in the kernel above): every read is one
  // of these plus a compile-time offset (buffer, half of the tile, key step)
  lds_ptr_t ka[KS];
#pragma unroll
  for (int j = 0; j < KS; ++j) ka[j] = (lds_ptr_t)&sm.k[0][0][0] + (uint32_t)(n * CPR + ((2 * j + h) ^ swz_k<CPR>(n))) * 16;
  const int li = lane & 15;
  const int vrow = (li >> 2) + 4 * h;
  const int vcol = 16 * ((lane >> 4) & 1) + 4 * (li & 3);
  lds_ptr_t va[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int c = (32 * dt + vcol) >> 3;
    va[dt] = (lds_ptr_t)&sm.v[0][0][0] + (uint32_t)((vrow * CPR + (c ^ swz_v<CPR>(vrow))) * 16 + (vcol & 7) * 2);
  }
  // opaque to the compiler, which would otherwise fold the offsets back into address arithmetic at every read
#pragma unroll
  for (int j = 0; j < KS; ++j) asm volatile("" : "+v"(ka[j]));
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) asm volatile("" : "+v"(va[dt]));

  const int tile_begin = split * p.tiles_per_split;
  int tile_end = min(tile_begin + p.tiles_per_split, p.num_tiles);
  if (!p.tp) {  // contiguous positions: tiles no row of this workgroup may see are skipped
    const int qpos_max = p.input_pos + min(mblk * BM + BM - 1, p.R - 1) / p.G;
    tile_end = min(tile_end, qpos_max / BN + 1);
    if (tile_end <= tile_begin) {
#pragma unroll
      for (int rb = 0; rb < NRB; ++rb)
        if (row_ok[rb]) {
          const int64_t prow = ((int64_t)split * p.B * p.Hkv + group) * p.R + row[rb];
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

  f32x16_t o[NO];
  zero_o<0>(o[0]);
  zero_o<1>(o[1]);
  zero_o<2>(o[2]);
  zero_o<3>(o[3]);
  if constexpr (NO == 8) {
    zero_o<4>(o[4]);
    zero_o<5>(o[5]);
    zero_o<6>(o[6]);
    zero_o<7>(o[7]);
  }
  // row sums of P, in fp32 from the unrounded values (the log-sum-exp feeds the score sums, which are held to
  // 1e-3): this lane's 16 keys of every step; the other half of the wavefront holds the other 16
  float lrow[NRB], m[NRB];
#pragma unroll
  for (int rb = 0; rb < NRB; ++rb) {
    lrow[rb] = 0.0f;
    m[rb] = -INFINITY;
  }
  const float slack = kSlackLog2 / p.c;

  f32x16_t sb[2][NRB];     // S of a step: [buffer][row block]
  u32x4_t pb[2][NRB][2];   // packed P of a step: [buffer][row block][key step of 16], the B operands of the second product

  TileSender ld;
  ld.init(p, sm, b, kvh, tid, tile_begin);

  constexpr int KBYTES = BN * CPR * 16;  // bytes of one K or V tile buffer
  // S(next) = K Q^T for 32 keys: key rows 32 MT .. of K buffer KBUF
  auto qk_all = [&](f32x16_t (&s)[NRB], auto kbuf_tag, auto mt_tag) {
    constexpr int OFF = decltype(kbuf_tag)::value * KBYTES + decltype(mt_tag)::value * 32 * CPR * 16;
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      const u32x4_t kk = *(const u32x4_t __attribute__((address_space(3)))*)(ka[j] + OFF);
#pragma unroll
      for (int rb = 0; rb < NRB; ++rb) {
        if (j == 0) mfma_s_first<F16>(s[rb], kk, qf[rb][0]);
        else mfma_s<F16>(s[rb], kk, qf[rb][j]);
      }
    }
  };
  // O += V^T P^T for the 32 keys of a step
  auto pv_all = [&](const u32x4_t (&pp)[NRB][2], auto vbuf_tag, auto mt_tag) {
    constexpr int OFF = decltype(vbuf_tag)::value * KBYTES + decltype(mt_tag)::value * 32 * CPR * 16;
    auto one = [&](auto dt_tag, int j) {
      constexpr int dt = decltype(dt_tag)::value;
      const lds_ptr_t vl = va[dt] + OFF + 16 * j * CPR * 16;
      const u32x2_t lo = lds_read_tr16(vl);
      const u32x2_t hi = lds_read_tr16(vl + 8 * CPR * 16);
      const u32x4_t vf = {lo[0], lo[1], hi[0], hi[1]};
      mfma_o<F16, dt * NRB>(o[dt * NRB], vf, pp[0][j]);
      if constexpr (NRB == 2) mfma_o<F16, dt * NRB + 1>(o[dt * NRB + 1], vf, pp[NRB - 1][j]);
    };
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      one(std::integral_constant<int, 0>{}, j);
      one(std::integral_constant<int, 1>{}, j);
      one(std::integral_constant<int, 2>{}, j);
      one(std::integral_constant<int, 3>{}, j);
    }
  };

  // Softmax state of the step about to run: m is the reference maximum its exponentials use, mc = m c, and alpha
  // is the factor that takes O and the row sums from the reference of the step before to this one (applied at
  // the end of the step, once the second product has added the P of the step before).
  float mc[NRB], alpha[NRB], mx[NRB];
#pragma unroll
  for (int rb = 0; rb < NRB; ++rb) {
    mc[rb] = 0.0f;
    alpha[rb] = 1.0f;
    mx[rb] = -INFINITY;
  }
  bool resc = false;
  // mask, row maxima and the rescaling decision for the S in sn: key rows 32 half .. of the tile in ring slot ts
  auto mask_next = [&](f32x16_t (&sn)[NRB], int ts, int half, int tpl) {  // tpl: sm.tp[ts][32 half + n]
    const unsigned hidden = (unsigned)__ballot(tpl > qpos_min_w);  // lanes 0..31: the step's 32 keys
    if (hidden) {
#pragma unroll
      for (int a = 0; a < 4; ++a)
        if ((hidden >> (8 * a)) & 0xffu) {
          const int4 tq = *(const int4*)&sm.tp[ts][half * 32 + 8 * a + 4 * h];
#pragma unroll
          for (int rb = 0; rb < NRB; ++rb) {
            if (tq.x > qpos[rb]) sn[rb][4 * a + 0] = -INFINITY;
            if (tq.y > qpos[rb]) sn[rb][4 * a + 1] = -INFINITY;
            if (tq.z > qpos[rb]) sn[rb][4 * a + 2] = -INFINITY;
            if (tq.w > qpos[rb]) sn[rb][4 * a + 3] = -INFINITY;
          }
        }
    }
  };
  auto decide = [&]() {
    bool need = false;
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) need |= mx[rb] > m[rb] + slack;
    resc = __any(need);
    if (resc) {
#pragma unroll
      for (int rb = 0; rb < NRB; ++rb) {
        const float m_new = fmaxf(m[rb], mx[rb]);
        const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
        alpha[rb] = fast_exp2((m[rb] - m_use) * p.c);
        lrow[rb] *= alpha[rb];  // the sums only hold steps before the one this decision is for
        m[rb] = m_new;
      }
    }
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) mc[rb] = (m[rb] == -INFINITY) ? 0.0f : m[rb] * p.c;
  };
  // The operand fragments of a step pass through a ring of RING registers, each read from LDS DIST fragments
  // before its first use (a fragment feeds NRB matrix instructions): fragments 0..7 are the K rows of the first
  // product, 8..15 the V rows of the second (8 + 4 j + dt), 16.. the first K rows of the step after.
  constexpr int RING = NRB == 2 ? 4 : 8;
  constexpr int DIST = RING - 1;
  u32x4_t fr[RING];

  // One step s = 2 (tile - tile_begin) + (K4 & 1), K4 = s mod 4: S(s) sits in sb[K4 & 1] with its mask, row
  // maxima and rescaling decision already taken. A wavefront issues in order, and a matrix instruction waits at
  // issue while the one before it occupies the matrix core (32 cycles), so vector work only overlaps the matrix
  // instruction that directly precedes it: the step is 16 NRB slots of one matrix instruction each, followed by a
  // slot's worth of vector work. The first half of the slots multiplies S(s+1) into sb[~K4 & 1], the second adds
  // V(s-1) P(s-1) to O; every slot also turns one element of S(s) into P(s), and a few of the later ones prepare
  // S(s+1). Tile t lives in LDS buffer (t - tile_begin) & 1; transfers start two steps before their tile is first
  // read and are published by the barrier in the first step of every tile.
  constexpr int NS = 16 * NRB;   // slots per step
  constexpr int NQK = 8 * NRB;   // slots of the first product
  auto step = [&](auto k4_tag, int tile) {
    constexpr int K4 = decltype(k4_tag)::value;
    constexpr int PAR = K4 & 1;
    constexpr int TBUF = (K4 >> 1) & 1;                 // LDS buffer of this step's tile
    constexpr int KBUF_N = ((K4 + 1) >> 1) & 1, MT_N = (K4 + 1) & 1;   // K rows of step s + 1
    constexpr int KBUF_NN = ((K4 + 2) >> 1) & 1, MT_NN = (K4 + 2) & 1;  // K rows of step s + 2
    constexpr int VBUF_P = ((K4 + 3) >> 1) & 1, MT_P = (K4 + 3) & 1;   // V rows of step s - 1
    constexpr int KOFF = KBUF_N * KBYTES + MT_N * 32 * CPR * 16;
    constexpr int KOFF_NN = KBUF_NN * KBYTES + MT_NN * 32 * CPR * 16;
    constexpr int VOFF = VBUF_P * KBYTES + MT_P * 32 * CPR * 16;
    f32x16_t (&s)[NRB] = sb[PAR];
    f32x16_t (&sn)[NRB] = sb[PAR ^ 1];
    pin_s(s);  // S(s), written by the step before, is read from here on, not earlier
    const int tsel = (tile - tile_begin) & 3;  // ring slot of this tile's token positions
    const bool has_next = K4 != 3 || tile + 1 < tile_end;  // tiles come in pairs: only the last step of a pair may be the last
    float pe = 0.0f, po = 0.0f;                // the pair of P elements to pack next
    int tpl_next = 0;                          // position of key n of the step after this one
    auto read_fragment = [&](auto f_tag) {
      constexpr int f = decltype(f_tag)::value;
      if constexpr (f < 8) {
        fr[f % RING] = *(const u32x4_t __attribute__((address_space(3)))*)(ka[f] + KOFF);
      } else if constexpr (f < 16) {
        const lds_ptr_t vl = va[f & 3] + VOFF + 16 * ((f - 8) >> 2) * CPR * 16;
        const u32x2_t lo = lds_read_tr16(vl);
        const u32x2_t hi = lds_read_tr16(vl + 8 * CPR * 16);
        fr[f % RING] = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
      } else {
        fr[f % RING] = *(const u32x4_t __attribute__((address_space(3)))*)(ka[f - 16] + KOFF_NN);
      }
    };
    auto slot = [&](auto sl_tag) {
      constexpr int SL = decltype(sl_tag)::value;
      constexpr int RB = SL % NRB;
      if constexpr (SL < NQK) {
        constexpr int J = SL / NRB;
        if constexpr (J == 0) mfma_s_first<F16>(sn[RB], fr[0], qf[RB][0]);
        else mfma_s<F16>(sn[RB], fr[J % RING], qf[RB][J]);
      } else {
        constexpr int I = (SL - NQK) / NRB, DTI = I & 3, J = I >> 2;
        mfma_o<F16, DTI * NRB + RB>(o[DTI * NRB + RB], fr[(8 + I) % RING], pb[PAR ^ 1][RB][J]);
      }
      if constexpr (RB == 0 && SL / NRB + DIST < 16) read_fragment(std::integral_constant<int, SL / NRB + DIST>{});
      if constexpr (SL == 1 && PAR == 1) {
        // V of the next tile into the buffer the second product left in the step before, K of the tile after it
        // into the buffer the first product left there
        ld.template send<false, TBUF ^ 1>(sm, tid, 0, tile_end);                // tile + 1
        ld.template send<true, TBUF>(sm, tid, (tsel + 2) & 3, tile_end);        // tile + 2
      }
      // P for key SL % 16 (register order) of row block SL / 16. Each result passes through an empty volatile
      // statement: without it the compiler sinks the whole computation below the step's last matrix instruction,
      // where nothing overlaps it. An exponential's result may not be read by the very next instruction, so the
      // row sum takes the element of the slot before, and a pair is packed one slot after its second element.
      if constexpr (SL >= 1) {
        lrow[(SL - 1) >> 4] += ((SL - 1) & 1) ? po : pe;
        asm volatile("" : "+v"(lrow[(SL - 1) >> 4]));
      }
      if constexpr (SL >= 2 && (SL & 1) == 0) {
        constexpr int E = (SL - 2) & 15, ERB = (SL - 2) >> 4;
        uint32_t pk = pack_pair<F16>(pe, po);
        asm volatile("" : "+v"(pk));
        pb[PAR][ERB][E >> 3][(E >> 1) & 3] = pk;
      }
      {
        constexpr int E = SL & 15, ERB = SL >> 4;
        float pv = fast_exp2(fmaf(s[ERB][E], p.c, -mc[ERB]));
        asm volatile("" : "+v"(pv));
        if constexpr (E & 1) po = pv;
        else pe = pv;
      }
      if constexpr (SL == 4 * NRB) tpl_next = sm.tp[PAR == 1 ? (tsel + 1) & 3 : tsel][(PAR ^ 1) * 32 + n];
      // S(s+1) is complete two slots after the last instruction of the first product: its mask and row maxima
      // go between the instructions of the second
      if constexpr (SL == NQK + 2) { if (has_next) mask_next(sn, PAR == 1 ? (tsel + 1) & 3 : tsel, PAR ^ 1, tpl_next); }
      if constexpr (SL == NQK + 5) { if (has_next) mx[0] = row_max_raw(sn[0]); }
      if constexpr (NRB == 2 && SL == NQK + 9) { if (has_next) mx[NRB - 1] = row_max_raw(sn[NRB - 1]); }
      if constexpr (NRB == 1) {  // two wavefronts per SIMD: the one further into its step goes first
        if constexpr (SL == NQK - 1) __builtin_amdgcn_s_setprio(1);
        if constexpr (SL == NQK + NQK / 2 - 1) __builtin_amdgcn_s_setprio(2);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (NRB == 1) __builtin_amdgcn_s_setprio(0);
    unroll_seq<0, NS>(slot);
    if constexpr (NRB == 1) __builtin_amdgcn_s_setprio(3);
    {
      lrow[NRB - 1] += po;
      uint32_t pk = pack_pair<F16>(pe, po);
      asm volatile("" : "+v"(pk));
      pb[PAR][NRB - 1][1][3] = pk;
    }
    pin_p(pb[PAR]);  // P(s) is complete here, a whole step before the matrix core reads it
    if constexpr (PAR == 0) {
      // one barrier per tile: what was sent in the second step of the tile before has landed (K and the positions
      // of the next tile, V of this one), and every wavefront is done with the buffers the next transfers take
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      ld.land(sm, tile + 1, tid, (tsel + 1) & 3, tile_end);
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
    }
    auto read_ahead = [&](auto i_tag) { read_fragment(std::integral_constant<int, 16 + decltype(i_tag)::value>{}); };
    unroll_seq<0, DIST>(read_ahead);
    __builtin_amdgcn_sched_barrier(0);
    if (resc) {  // O (now including step s - 1) moves to the reference maximum of P(s)
      settle_o(o);  // the last matrix instructions have to leave O first
      scale_o<0>(o[0], alpha[0]);
      scale_o<1>(o[1], alpha[1 % NRB]);
      scale_o<2>(o[2], alpha[2 % NRB]);
      scale_o<3>(o[3], alpha[3 % NRB]);
      if constexpr (NO == 8) {
        scale_o<4>(o[4], alpha[0]);
        scale_o<5>(o[5], alpha[1 % NRB]);
        scale_o<6>(o[6], alpha[0]);
        scale_o<7>(o[7], alpha[1 % NRB]);
      }
      resc = false;
    }
    if (has_next) decide();
    __builtin_amdgcn_sched_barrier(0);  // nothing of this step moves into the next one
  };

  // prologue: first tile into buffer 0, K of the second into buffer 1, S(0) and its preparation. The first step
  // multiplies the second half of V buffer 1 by P = 0: the buffer is cleared, since 0 x (whatever LDS held) may be NaN.
  ld.template send<true, 0>(sm, tid, 0, tile_end);
  ld.template send<false, 0>(sm, tid, 0, tile_end);
  ld.template send<true, 1>(sm, tid, 1, tile_end);
  {
    const u32x4_t z = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < BN * CPR / 256; ++i) (&sm.v[1][0][0])[tid + 256 * i] = z;
  }
#pragma unroll
  for (int rb = 0; rb < NRB; ++rb)
#pragma unroll
    for (int j = 0; j < 2; ++j) pb[1][rb][j] = u32x4_t{0u, 0u, 0u, 0u};
  __builtin_amdgcn_s_waitcnt(0x0F70);
  ld.land(sm, tile_begin, tid, 0, tile_end);
  __syncthreads();
  constexpr std::integral_constant<int, 0> I0{};
  constexpr std::integral_constant<int, 1> I1{};
  constexpr std::integral_constant<int, 2> I2{};
  constexpr std::integral_constant<int, 3> I3{};
  qk_all(sb[0], I0, I0);
#pragma unroll
  for (int j = 0; j < DIST; ++j) fr[j] = *(const u32x4_t __attribute__((address_space(3)))*)(ka[j] + 32 * CPR * 16);  // K rows of step 1
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // S(0) is read right away
  pin_s(sb[0]);
  pin_p(pb[1]);
  mask_next(sb[0], 0, 0, sm.tp[0][n]);
#pragma unroll
  for (int rb = 0; rb < NRB; ++rb) mx[rb] = row_max_raw(sb[0][rb]);
  decide();
  // Tiles alternate between the two LDS buffers and the step templates cover a pair of them. A walk over an odd
  // number of tiles ends with a tile that is not there: nothing is transferred for it, all its positions are
  // hidden, so its P is zero and the stale (finite) V rows it meets add nothing.
  int t = tile_begin;
  do {
    step(I0, t);
    step(I1, t);
    step(I2, t + 1);
    step(I3, t + 1);
    t += 2;
  } while (t < tile_end);
  pv_all(pb[1], I1, I1);  // P of the last step: second half of the tile in buffer 1
  settle_o(o);            // O is read by the vector ALU next
  // from the fixed accumulation registers into ordinary ones (the compiler may not take parts of a fixed register)
#pragma unroll
  for (int i = 0; i < NO; ++i) asm volatile("" : "+v"(o[i]));

  // ---- epilogue -----------------------------------------------------------------------------
  // The row coordinates are taken again from the lane number here: held across the loop they would occupy
  // registers the loop needs.
  int tid_e = threadIdx.x;
  asm volatile("" : "+v"(tid_e));
  const int h_e = (tid_e >> 5) & 1;
#pragma unroll
  for (int rb = 0; rb < NRB; ++rb) {
    const float lt = sum_halves(lrow[rb]);
    const int row_e = mblk * BM + (tid_e >> 6) * 32 * NRB + rb * 32 + (tid_e & 31);
    if (row_e >= p.R) continue;
    const int qi_e = row_e / p.G, g_e = row_e % p.G;
    if (p.num_splits == 1) {
      const float inv = lt > 0.0f ? 1.0f / lt : 0.0f;
      uint16_t* op = p.o + b * p.o_sb + (int64_t)(kvh * p.G + g_e) * p.o_sh + (int64_t)qi_e * p.o_st;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const f32x16_t& ob = o[dt * NRB + rb];
          u32x2_t w2;
          w2[0] = pack_pair<F16>(ob[4 * a] * inv, ob[4 * a + 1] * inv);
          w2[1] = pack_pair<F16>(ob[4 * a + 2] * inv, ob[4 * a + 3] * inv);
          *(u32x2_t*)(op + dt * 32 + 8 * a + 4 * h_e) = w2;
        }
      if (p.lse && h_e == 0) p.lse[((int64_t)b * p.q_len + qi_e) * p.Hq + kvh * p.G + g_e] = m[rb] * p.c + fast_log2(lt);
    } else {
      const int64_t prow = ((int64_t)split * p.B * p.Hkv + group) * p.R + row_e;
      float* po = p.part_o + prow * D;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const f32x16_t& ob = o[dt * NRB + rb];
          f32x4_t w4 = {ob[4 * a], ob[4 * a + 1], ob[4 * a + 2], ob[4 * a + 3]};
          *(f32x4_t*)(po + dt * 32 + 8 * a + 4 * h_e) = w4;
        }
      if (h_e == 0) {
        p.part_ml[prow * 2] = m[rb] * p.c;
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

// Three kernels serve plain rows with D = 128: the 32-row kernel above ("classic": the compiler schedules the
// step), and the slot kernel with 32 or 64 rows per wavefront ("slots32": two workgroups per compute unit,
// "slots64": one; 64 rows need a workgroup's worth of rows per (batch, KV head) pair). KVX_PREFILL_KERNEL in the
// environment (looked up at every call) picks one by name; without it the default below is used.
enum PrefillVariant { PF_CLASSIC = 0, PF_SLOTS32 = 1, PF_SLOTS64 = 2 };
constexpr int PF_DEFAULT = PF_CLASSIC;
int prefill_variant(const kvx_sdpa_args& a) {
  if (a.D != 128 || !kv_is_plain(a.kv_dtype)) return PF_CLASSIC;
  int v = PF_DEFAULT;
  if (const char* e = getenv("KVX_PREFILL_KERNEL")) {
    if (!strcmp(e, "classic")) v = PF_CLASSIC;
    else if (!strcmp(e, "slots32")) v = PF_SLOTS32;
    else if (!strcmp(e, "slots64")) v = PF_SLOTS64;
  }
  if (v == PF_SLOTS64 && (int64_t)a.q_len * (a.Hq / a.Hkv) < W64_BM) v = PF_SLOTS32;
  return v;
}

int pick_splits(const kvx_sdpa_args& a, int m_blocks, int num_tiles) {
  if (a.num_splits > 0) return min(a.num_splits, num_tiles);
  // Aim for one resident round of workgroups (2 per compute unit, 1 with the uint8 cache): more
  // splits only add partials to write, merge and re-read. At least 8 key tiles per split.
  const int64_t base = (int64_t)a.B * a.Hkv * m_blocks;
  const int target = ((kv_is_plain(a.kv_dtype) && a.D <= 128 && prefill_variant(a) != PF_SLOTS64) ? 2 : 1) * num_cus();
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
  const int bm = prefill_variant(a) == PF_SLOTS64 ? W64_BM : 32 * nwaves(a.kv_dtype);
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
int launch_t(PrefillParams& p, hipStream_t st, int variant = PF_CLASSIC) {
  dim3 grid(p.B * p.Hkv, p.m_blocks, p.num_splits);
  if constexpr (D == 128 && kv_is_plain(KV)) {
    if (variant == PF_SLOTS64) hipLaunchKernelGGL((sdpa_prefill_slots_kernel<KV, 2>), grid, dim3(256), 0, st, p);
    else if (variant == PF_SLOTS32) hipLaunchKernelGGL((sdpa_prefill_slots_kernel<KV, 1>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((sdpa_prefill_kernel<D, KV>), grid, dim3(64 * nwaves(KV)), 0, st, p);
  } else {
    hipLaunchKernelGGL((sdpa_prefill_kernel<D, KV>), grid, dim3(64 * nwaves(KV)), 0, st, p);
  }
  KVX_HIP(hipGetLastError());
  if (p.num_splits > 1) {
    constexpr int ROWS = 256 / (D / 4);
    const int64_t total_rows = (int64_t)p.B * p.Hkv * p.R;
    hipLaunchKernelGGL((sdpa_prefill_merge_kernel<D, KV == KVX_KV_F16>), dim3((unsigned)((total_rows + ROWS - 1) / ROWS)), dim3(256), 0, st, p);
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
  if (a.D == 128) {
    if (a.kv_dtype == KVX_KV_U4) return launch_t<128, KVX_KV_U4>(p, st);
    if (a.kv_dtype == KVX_KV_F16) return launch_t<128, KVX_KV_F16>(p, st, prefill_variant(a));
    return a.kv_dtype == KVX_KV_U8 ? launch_t<128, KVX_KV_U8>(p, st) : launch_t<128, KVX_KV_BF16>(p, st, prefill_variant(a));
  }
  if (a.D == 64) {
    if (a.kv_dtype == KVX_KV_U4) return launch_t<64, KVX_KV_U4>(p, st);
    if (a.kv_dtype == KVX_KV_F16) return launch_t<64, KVX_KV_F16>(p, st);
    return a.kv_dtype == KVX_KV_U8 ? launch_t<64, KVX_KV_U8>(p, st) : launch_t<64, KVX_KV_BF16>(p, st);
  }
  if (a.D == 256 && kv_is_plain(a.kv_dtype))
    return a.kv_dtype == KVX_KV_F16 ? launch_t<256, KVX_KV_F16>(p, st) : launch_t<256, KVX_KV_BF16>(p, st);
  return set_error(KVX_ERR_UNSUPPORTED, "kvx_sdpa_prefill: head size %d not in {64, 128, 256} (quantised stores: {64, 128})", a.D);
}

}  // namespace kvx
