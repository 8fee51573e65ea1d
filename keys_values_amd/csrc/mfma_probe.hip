// What the matrix cores of a gfx950 device sustain, and what a wavefront can issue beside them: the ceilings the
// attention kernels are measured against. A stand-alone program (built next to the library, run by
// `bench.py --workload ceiling`): every row launches one kernel over the whole device and reports the shader
// clock it ran at (cycle counter / 100 MHz wall counter), cycles per round and, for matrix work, TFLOP/s.
//
//   rounds of one v_mfma_f32_32x32x16_bf16 (32768 FLOP per lane group, 32 cycles of the matrix core) plus
//   - nothing, with random or all-zero operands (the clock follows the power the operands draw);
//   - K independent v_fma_f32, or 2 v_exp_f32: does vector work fit beside the matrix instruction;
//   - the vector work of one attention slot (fma, exp, half a bf16 pack) and an LDS fragment read;
//   - a 1 KB transfer from L2 straight into LDS (global_load_lds_dwordx4) every K rounds: what the K / V tile
//     stream of the attention kernels (one transfer per 4 matrix instructions and wavefront) costs;
//   - everything the attention kernel issues per matrix instruction, as its counters give it (4.6 vector instructions:
//     fma, exp, add, half a pack, a third of a max3, one more; 1.5 LDS reads of 8 bytes per lane; the tile stream),
//     with no dependence of one round on another and no barrier: what that instruction mix alone allows;
//   - the same for the score-sum kernel (two elements per matrix instruction: fma, exp, add each; a 16-byte LDS read per two);
//   and the same vector work alone, at one and two wavefronts per SIMD: the issue rate of a single wavefront.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

#define CK(x)                                                                \
  do {                                                                       \
    hipError_t e_ = (x);                                                     \
    if (e_ != hipSuccess) {                                                  \
      printf("error: %s at line %d\n", hipGetErrorString(e_), __LINE__);     \
      return 1;                                                              \
    }                                                                        \
  } while (0)

enum Mix { NONE = 0, FMA = 1, EXP = 2, SLOT = 3, DMA = 4, ATT = 5, SSUM = 6 };
constexpr int ROUNDS = 16;  // rounds per loop iteration

// MF: issue the matrix instruction; MIX / K: the vector work of a round; RANDOM: operand bits
template <bool MF, int MIX, int K>
__global__ __launch_bounds__(256) void probe_kernel(const uint32_t* rnd, float* out, long long* cyc, int iters, int random, const char* stream) {
  __shared__ u32x4 sm[1024];
  __shared__ u32x4 landing[4][4][64];  // per wavefront: four 1 KB landing places for the transfers
  for (int i = threadIdx.x; i < 1024; i += 256) {  // operands read from LDS are as random as those held in registers
    u32x4 t = *(const u32x4*)(rnd + ((i * 4 + blockIdx.x * 16) & 4092));
    for (int e = 0; e < 4; ++e) t[e] = random ? ((t[e] & 0x807f807fu) | 0x3f003f00u) : 0u;
    sm[i] = t;
  }
  __syncthreads();
  u32x4 ar = *(const u32x4*)(rnd + ((threadIdx.x * 4 + blockIdx.x * 64) & 4092));
  u32x4 br = *(const u32x4*)(rnd + ((threadIdx.x * 4 + 2048 + blockIdx.x * 32) & 4092));
  for (int i = 0; i < 4; ++i) {  // random sign and mantissa, exponent near 0; or zeros
    ar[i] = random ? ((ar[i] & 0x807f807fu) | 0x3f003f00u) : 0u;
    br[i] = random ? ((br[i] & 0x807f807fu) | 0x3f003f00u) : 0u;
  }
  float v[8];
  for (int i = 0; i < 8; ++i) v[i] = 0.25f + 0.001f * (float)((threadIdx.x + i) & 63);
  float w = 1.0001f, mc = 0.5f, pe = 0.0f;
  uint32_t pk = 0;
  f32x16 acc[4];
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.0f;
  u32x4 frag = ar;
  u32x4 ring[4] = {ar, br, ar, br};
  const u32x4 __attribute__((address_space(3)))* lp = (const u32x4 __attribute__((address_space(3)))*)sm + ((threadIdx.x & 63) ^ ((threadIdx.x >> 2) & 15));
  // transfers walk a 256 KB window of `stream` shared by the workgroups of one XCD (workgroup i runs on XCD i % 8),
  // as the row blocks of one KV head share its K / V tiles: L2 hits after the first pass
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(&landing[wave][0][0]));
  const char* window = stream + (size_t)(blockIdx.x & 7) * 262144;
  uint32_t voff = (threadIdx.x & 63) * 16 + wave * 65536;
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < ROUNDS; ++j) {
      if (MF) acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, MIX == ATT ? ring[j & 3] : (MIX == SSUM ? ring[(j / 2) & 3] : (MIX == SLOT ? frag : ar))), __builtin_bit_cast(bf16x8, br), acc[j & 3], 0, 0, 0);
      if (MIX == FMA) {
#pragma unroll
        for (int i = 0; i < K; ++i) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v[i % 8]) : "v"(w), "v"(v[(i + 3) % 8]));
      }
      if (MIX == EXP) {
#pragma unroll
        for (int i = 0; i < K; ++i) asm volatile("v_exp_f32 %0, %0" : "+v"(v[i % 8]));
      }
      if (MIX == SLOT) {
        if ((j & 1) == 0) frag = lp[64 * ((j >> 1) & 7)];
        float t = __builtin_amdgcn_exp2f(__builtin_fmaf(v[j & 7], w, -mc));
        asm volatile("" : "+v"(t));
        if (j & 1) asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(pk) : "v"(pe), "v"(t));
        else pe = t;
      }
      if (MIX == ATT) {
        const u32x2 __attribute__((address_space(3)))* lp2 = (const u32x2 __attribute__((address_space(3)))*)lp;
        // operands are read three rounds before the matrix instruction that takes them
        u32x2 f0 = lp2[128 * (j & 7)];
        ring[(j + 3) & 3][0] = f0[0];
        ring[(j + 3) & 3][1] = f0[1];
        if (j & 1) {
          u32x2 f1 = lp2[128 * (j & 7) + 1024];
          ring[(j + 3) & 3][2] = f1[0];
          ring[(j + 3) & 3][3] = f1[1];
        }
        float t = __builtin_amdgcn_exp2f(__builtin_fmaf(v[j & 7], w, -mc));
        asm volatile("" : "+v"(t));
        float l = v[(j + 1) & 7] + t;
        asm volatile("" : "+v"(l));
        v[(j + 1) & 7] = l * 0.5f;
        if (j & 1) asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(pk) : "v"(pe), "v"(t));
        else pe = t;
        if (j % 3 == 0) asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(mc) : "v"(t), "v"(pe));
      }
      if (MIX == SSUM) {  // the score-sum kernel: two elements per matrix instruction (fma, exp, add each), a 16-byte LDS read per two
        if ((j & 1) == 0) ring[(j / 2 + 3) & 3] = lp[64 * ((j >> 1) & 7)];
        float t0 = __builtin_amdgcn_exp2f(__builtin_fmaf(v[j & 7], w, -mc));
        float t1 = __builtin_amdgcn_exp2f(__builtin_fmaf(v[(j + 1) & 7], w, -mc));
        asm volatile("" : "+v"(t0), "+v"(t1));
        pe += t0 + t1;
      }
      if ((MIX == DMA || MIX == ATT) && j % (MIX == ATT ? 4 : K) == 0) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds0 + 1024u * ((j / K) & 3)), "v"(voff), "s"(window) : "memory", "m0");
        voff = (voff & 0xffff0000u) | ((voff + 1024u) & 0xffffu);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // the transfers of the iteration before have landed; those just issued stay in flight (a kernel that double-buffers its tiles waits like this)
    if (MIX == DMA || MIX == ATT) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(ROUNDS / (MIX == ATT ? 4 : (K > 0 ? K : 1))) : "memory");
    if (MIX == ATT) mc = 0.5f;
    if (MF && (it & 63) == 63)
      for (int j = 0; j < 4; ++j)
        for (int i = 0; i < 16; ++i) acc[j][i] *= 1e-30f;  // keeps the sums finite
    if (MIX == SLOT) br[0] ^= pk & 1u;
  }
  const long long c1 = clock64(), w1 = wall_clock64();
  float s = pe + (float)pk + __uint_as_float(frag[0]) + __uint_as_float(ring[0][0] ^ ring[1][1] ^ ring[2][2] ^ ring[3][3]) + ((MIX == DMA || MIX == ATT) ? __uint_as_float(landing[wave][1][threadIdx.x & 63][0]) : 0.0f);
  for (int i = 0; i < 8; ++i) s += v[i];
  for (int j = 0; j < 4; ++j)
    for (int i = 0; i < 16; ++i) s += acc[j][i];
  out[blockIdx.x * 256 + threadIdx.x] = s;
  if (threadIdx.x == 0) {
    cyc[2 * blockIdx.x] = c1 - c0;
    cyc[2 * blockIdx.x + 1] = w1 - w0;
  }
}

static uint32_t* g_rnd;
static float* g_out;
static long long* g_cyc;
static char* g_stream;
static int g_cus;

template <bool MF, int MIX, int K>
int run(const char* name, int waves_per_simd, int random) {
  const int iters = 3000, blocks = g_cus * waves_per_simd;  // a workgroup is four wavefronts, one per SIMD
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  hipLaunchKernelGGL((probe_kernel<MF, MIX, K>), dim3(blocks), dim3(256), 0, 0, g_rnd, g_out, g_cyc, iters, random, g_stream);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0));
  hipLaunchKernelGGL((probe_kernel<MF, MIX, K>), dim3(blocks), dim3(256), 0, 0, g_rnd, g_out, g_cyc, iters, random, g_stream);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  static long long hh[8192];
  CK(hipMemcpy(hh, g_cyc, 16 * blocks, hipMemcpyDeviceToHost));
  double sc = 0, wc = 0;
  for (int i = 0; i < blocks; ++i) {
    sc += (double)hh[2 * i];
    wc += (double)hh[2 * i + 1];
  }
  const double rounds = (double)iters * ROUNDS;
  const double tflops = MF ? blocks * 4.0 * rounds * 32768.0 / (ms * 1e-3) / 1e12 : 0.0;
  printf("%-46s %d wave/SIMD  %s  %6.3f ms  %4.2f GHz  %5.1f cycles/round/wave  %7.1f TFLOP/s\n", name, waves_per_simd, random ? "random" : "zeros ", ms,
         sc / wc * 0.1, sc / blocks / rounds, tflops);
  return 0;
}

int main() {
  hipDeviceProp_t prop;
  CK(hipGetDeviceProperties(&prop, 0));
  g_cus = prop.multiProcessorCount;
  printf("device: %s, %d compute units\n", prop.gcnArchName, g_cus);
  CK(hipMalloc(&g_rnd, 16384));
  CK(hipMalloc(&g_out, 8192 * 256 * 4));
  CK(hipMalloc(&g_cyc, 8192 * 16));
  CK(hipMalloc(&g_stream, (size_t)8 * 262144));
  CK(hipMemset(g_stream, 0x3c, (size_t)8 * 262144));
  static uint32_t h[4096];
  srand(5);
  for (auto& x : h) x = ((uint32_t)rand() << 16) ^ (uint32_t)rand();
  CK(hipMemcpy(g_rnd, h, sizeof(h), hipMemcpyHostToDevice));
  int rc = 0;
  for (int wps = 1; wps <= 2; ++wps) {
    rc |= run<true, NONE, 0>("matrix instruction only", wps, 1);
    rc |= run<true, NONE, 0>("matrix instruction only", wps, 0);
    rc |= run<true, FMA, 3>("matrix instruction + 3 fma", wps, 1);
    rc |= run<true, FMA, 6>("matrix instruction + 6 fma", wps, 1);
    rc |= run<true, FMA, 8>("matrix instruction + 8 fma", wps, 1);
    rc |= run<true, EXP, 2>("matrix instruction + 2 exp", wps, 1);
    rc |= run<true, SLOT, 0>("matrix instruction + fma, exp, pack/2, LDS read/2", wps, 1);
    rc |= run<true, DMA, 8>("matrix instruction + 1 KB L2->LDS per 8", wps, 1);
    rc |= run<true, DMA, 4>("matrix instruction + 1 KB L2->LDS per 4", wps, 1);
    rc |= run<true, DMA, 2>("matrix instruction + 1 KB L2->LDS per 2", wps, 1);
    rc |= run<true, ATT, 0>("matrix instruction + the attention kernel's mix", wps, 1);
    rc |= run<true, SSUM, 0>("matrix instruction + the score-sum kernel's mix", wps, 1);
    rc |= run<false, FMA, 6>("6 fma", wps, 1);
    rc |= run<false, EXP, 2>("2 exp", wps, 1);
    rc |= run<false, SLOT, 0>("fma, exp, pack/2, LDS read/2", wps, 1);
  }
  return rc;
}
