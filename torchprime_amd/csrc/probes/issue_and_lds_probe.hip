// A stand-alone measurement program (not part of libtprime_hip.so): the facts about gfx950 that the attention
// kernels' LDS layouts and slot schedules rest on.
//   (1) LDS read rates of ds_read_b128 / ds_read_b64 / ds_read_b64_tr_b16 with nothing else in the instruction
//       stream, for the address patterns the kernels use (MFMA fragment reads and transposing reads of a dense
//       64 x 128 16-bit tile under two XOR swizzles);
//   (2) one wave per SIMD: cycles per MFMA when every MFMA comes with one 16-byte fragment read (or two transposing
//       reads) and n vector-ALU instructions / exponentials: what an instruction slot costs;
//   (3) two waves per SIMD: an evenly mixed instruction stream against phase-separated streams (one group of waves
//       issues MFMAs while the other does its element-wise work, with and without barriers and wave priorities).
//   (4) accumulators in architectural or accumulation registers, chains of dependent MFMAs, independent FMAs under them;
//   (5) FMAs that read MFMA results and feed MFMA operands (build with -mllvm -amdgpu-mfma-vgpr-form=1 for this part:
//       with the compiler's default form the accumulators are copied between the register halves around every read);
//   (6) MFMAs alone on normal-distributed and on zero operands: the clock the part sustains, and whether the order of
//       the MFMAs (re-use of an operand across consecutive ones) changes it.
// Build and run:  make -C torchprime_amd/csrc probes && torchprime_amd/csrc/build/issue_and_lds_probe
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstring>
#include <cstdlib>
#include <cstdio>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
#define LDSP(T, p) ((__attribute__((address_space(3))) T*)(p))

template <typename F> float timeit(F f, int reps = 3) {
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  f(); CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0)); for (int i = 0; i < reps; i++) f(); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
  float ms; CK(hipEventElapsedTime(&ms, e0, e1)); return ms / reps;
}

// ---- (1) read rate.  KIND 0: ds_read_b128, 1: ds_read_b64, 2: ds_read_b64_tr_b16
// PAT 0: contiguous; 1: fragment pattern of a 64x128 bf16 tile with swizzle f(row)=row&15 (b128: row=ln, chunk 2ks+g;
// tr: 4 rows x 64 B per 32 lanes); 2: same with the rotated swizzle ((row&3)<<2)|((row>>2)&3)
template <int KIND, int PAT>
__global__ __launch_bounds__(256) void rd(float* out, int iters, long long* cyc) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[65536];
  const int t = threadIdx.x, l = t & 63;
  for (int i = t; i < 16384; i += 256) ((unsigned*)lds)[i] = i;
  __syncthreads();
  unsigned base;
  auto swz = [&](int row) { return PAT == 1 ? (row & 15) : (((row & 3) << 2) | ((row >> 2) & 3)); };
  if (PAT == 0) base = l * (KIND == 0 ? 16 : 8);
  else if (KIND == 0) { const int ln = l & 31, g = l >> 5; base = ln * 256 + ((g ^ swz(ln)) << 4); }
  else {
    const int g = l >> 5, mp = (l & 15) >> 2, row = 4 * g + mp;
    const int chunk = 2 * ((l >> 4) & 1) + ((l >> 1) & 1);
    base = row * 256 + ((chunk ^ swz(row)) << 4) + 8 * (l & 1);
  }
  u32x4 acc = {0, 0, 0, 0};
  long long t0 = __builtin_readcyclecounter();
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int j = 0; j < 16; j++) {
      const unsigned a = base + (j & 3) * 16384 + (j >> 2) * 2048;  // immediates
      if (KIND == 0) { u32x4 v = *(u32x4*)(lds + a); asm volatile("" :: "v"(v)); }
      else if (KIND == 1) { u32x2 v = *(u32x2*)(lds + a); asm volatile("" :: "v"(v)); }
      else { s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDSP(s16x4, lds + a)); asm volatile("" :: "v"(v)); }
    }
  }
  long long t1 = __builtin_readcyclecounter();
  out[blockIdx.x * 256 + t] = (float)acc.x;
  if (blockIdx.x == 0 && t == 0) cyc[0] = t1 - t0;
}

// ---- (2) one wave per SIMD (256 threads, 1 block per CU): per MFMA RK reads + NV valu (+ NE exps)
// RK 0: none, 1: one b128, 2: two tr b64
template <int RK, int NV, int NE>
__global__ __launch_bounds__(256) void one(float* out, int iters, long long* cyc) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[65536];
  const int t = threadIdx.x, l = t & 63;
  for (int i = t; i < 16384; i += 256) ((unsigned*)lds)[i] = 0x3c003c00u;
  __syncthreads();
  bf16x8 b; for (int e = 0; e < 8; e++) b[e] = (__bf16)1.0f;
  f32x16 c[4]; for (int i = 0; i < 4; i++) for (int v = 0; v < 16; v++) c[i][v] = 0.f;
  float x[8]; for (int i = 0; i < 8; i++) x[i] = l * 0.001f + i;
  const unsigned base = l * 16, base8 = l * 8;
  constexpr int AH = 4;
  u32x4 fr[AH];
  for (int i = 0; i < AH; i++) fr[i] = *(u32x4*)(lds + base + i * 1024);
  long long t0 = __builtin_readcyclecounter();
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int j = 0; j < 16; j++) {
      c[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fr[j % AH]), b, c[j & 3], 0, 0, 0);
      if (RK == 1) fr[j % AH] = *(u32x4*)(lds + base + ((j + AH) & 31) * 1024);
      if (RK == 2) {
        s16x4 v0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDSP(s16x4, lds + base8 + ((j + AH) & 31) * 1024));
        s16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDSP(s16x4, lds + base8 + ((j + AH) & 31) * 1024 + 512));
        u32x2 a0 = __builtin_bit_cast(u32x2, v0), a1 = __builtin_bit_cast(u32x2, v1);
        fr[j % AH] = u32x4{a0.x, a0.y, a1.x, a1.y};
      }
#pragma unroll
      for (int k = 0; k < NV; k++) x[(j + k) % 8] = x[(j + k) % 8] * 0.999f + 0.5f;
#pragma unroll
      for (int k = 0; k < NE; k++) x[(j + k + 3) % 8] = __builtin_amdgcn_exp2f(x[(j + k + 3) % 8]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  long long t1 = __builtin_readcyclecounter();
  float s = 0; for (int i = 0; i < 4; i++) s += c[i][0]; for (int i = 0; i < 8; i++) s += x[i];
  out[blockIdx.x * 256 + t] = s;
  if (blockIdx.x == 0 && t == 0) cyc[0] = t1 - t0;
}

// ---- (3) two waves per SIMD (512 threads).  Per tile and wave: NM MFMAs (each with one b128 fragment read, ring of 4)
// and NM * VPM valu + NM * EPM exps that depend on the MFMA results of the tile and feed the next tile's B operands.
// MODE 0: evenly mixed, barrier per tile.  1: evenly mixed, no barrier.  2: phases [M][V], groups (waves 0-3 / 4-7) in
// opposite phases, barrier after each phase.  3: phases, both groups in the same phase, barrier after each phase.
// 4: phases, opposite, no barriers at all (free running, group 1 starts with its V phase).
// 5: like 2 with s_setprio 1 around the MFMA phase
template <int MODE, int NM, int VPM, int EPM>
__global__ __launch_bounds__(512) void two(float* out, int iters, long long* cyc) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[65536];
  const int t = threadIdx.x, l = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
  for (int i = t; i < 16384; i += 512) ((unsigned*)lds)[i] = 0x3c003c00u;
  __syncthreads();
  bf16x8 b; for (int e = 0; e < 8; e++) b[e] = (__bf16)1.0f;
  f32x16 c[4]; for (int i = 0; i < 4; i++) for (int v = 0; v < 16; v++) c[i][v] = 0.f;
  float x[8]; for (int i = 0; i < 8; i++) x[i] = l * 0.001f + i;
  const unsigned base = l * 16 + (w & 3) * 8192;
  constexpr int AH = 4;
  u32x4 fr[AH];
  for (int i = 0; i < AH; i++) fr[i] = *(u32x4*)(lds + base + i * 1024);
  auto mphase = [&]() {
#pragma unroll
    for (int j = 0; j < NM; j++) {
      c[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fr[j % AH]), b, c[j & 3], 0, 0, 0);
      fr[j % AH] = *(u32x4*)(lds + base + ((j + AH) & 7) * 1024);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto vwork = [&](int j) {
#pragma unroll
    for (int k = 0; k < VPM; k++) x[(j + k) % 8] = x[(j + k) % 8] * 0.999f + 0.5f;
#pragma unroll
    for (int k = 0; k < EPM; k++) x[(j + k + 3) % 8] = __builtin_amdgcn_exp2f(x[(j + k + 3) % 8]);
  };
  auto vphase = [&]() {
    // depends on the MFMA results, produces the next B operand
    x[0] += c[0][0] * 1e-30f; x[1] += c[1][3] * 1e-30f; x[2] += c[2][5] * 1e-30f; x[3] += c[3][7] * 1e-30f;
#pragma unroll
    for (int j = 0; j < NM; j++) { vwork(j); }
    b[0] = (__bf16)(x[0] * 1e-30f + 1.f);
    __builtin_amdgcn_sched_barrier(0);
  };
  const bool grp1 = w >= 4;
  long long t0 = __builtin_readcyclecounter();
  if (MODE == 4 && grp1) vphase();
  for (int i = 0; i < iters; i++) {
    if (MODE <= 1) {
      x[0] += c[0][0] * 1e-30f;
#pragma unroll
      for (int j = 0; j < NM; j++) {
        c[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fr[j % AH]), b, c[j & 3], 0, 0, 0);
        fr[j % AH] = *(u32x4*)(lds + base + ((j + AH) & 7) * 1024);
        vwork(j);
        __builtin_amdgcn_sched_barrier(0);
      }
      b[0] = (__bf16)(x[0] * 1e-30f + 1.f);
      if (MODE == 0) __syncthreads();
    } else if (MODE == 2 || MODE == 5) {
      if (!grp1) { if (MODE == 5) __builtin_amdgcn_s_setprio(1); mphase(); if (MODE == 5) __builtin_amdgcn_s_setprio(0); } else vphase();
      __syncthreads();
      if (!grp1) vphase(); else { if (MODE == 5) __builtin_amdgcn_s_setprio(1); mphase(); if (MODE == 5) __builtin_amdgcn_s_setprio(0); }
      __syncthreads();
    } else if (MODE == 3) {
      mphase();
      __syncthreads();
      vphase();
      __syncthreads();
    } else {
      mphase();
      vphase();
    }
  }
  long long t1 = __builtin_readcyclecounter();
  float s = 0; for (int i = 0; i < 4; i++) s += c[i][0]; for (int i = 0; i < 8; i++) s += x[i];
  out[blockIdx.x * 512 + t] = s;
  if (blockIdx.x == 0 && l == 0) cyc[w] = t1 - t0;
}

// ---- (4) where the accumulators live: NW waves per SIMD, per MFMA NV independent FMAs; the MFMA is an asm statement
// whose accumulator is pinned to the architectural registers (ACC 0) or to the accumulation registers (ACC 1);
// CHAIN accumulators in rotation (1: every MFMA depends on the one before, as the k-steps of one product do)
template <int ACC, int CHAIN, int NV, int THREADS>
__global__ __launch_bounds__(THREADS) void acc_kind(float* out, int iters, long long* cyc) {
  const int t = threadIdx.x, l = t & 63;
  bf16x8 a, b;
  for (int e = 0; e < 8; e++) { a[e] = (__bf16)(1.0f + l * 0.001f); b[e] = (__bf16)1.0f; }
  f32x16 c[4];
  for (int i = 0; i < 4; i++) for (int v = 0; v < 16; v++) c[i][v] = 0.f;
  float x[8];
  for (int i = 0; i < 8; i++) x[i] = l * 0.001f + i;
  if (ACC) { asm volatile("" : "+a"(c[0]), "+a"(c[1]), "+a"(c[2]), "+a"(c[3])); }
  long long t0 = __builtin_readcyclecounter();
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int j = 0; j < 16; j++) {
      if (ACC) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c[j % CHAIN]) : "v"(a), "v"(b));
      else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c[j % CHAIN]) : "v"(a), "v"(b));
#pragma unroll
      for (int k = 0; k < NV; k++) x[(j + k) % 8] = x[(j + k) % 8] * 0.999f + 0.5f;
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  long long t1 = __builtin_readcyclecounter();
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // past the last MFMA's latency before ordinary instructions read c
  if (ACC) { asm volatile("" : "+a"(c[0]), "+a"(c[1]), "+a"(c[2]), "+a"(c[3])); }
  float s = 0;
  for (int i = 0; i < 4; i++) s += c[i][0];
  for (int i = 0; i < 8; i++) s += x[i];
  out[blockIdx.x * THREADS + t] = s;
  if (blockIdx.x == 0 && t == 0) cyc[0] = t1 - t0;
}

// ---- (5) what the vector-ALU work reads: per MFMA (compiler-known, four accumulators in rotation) NV FMAs that
// read x only (SRC 0), or one value each of the accumulator written two MFMAs earlier (SRC 1), or that and feed the
// next MFMAs' B operand through a conversion (SRC 2: the MFMA -> VALU -> MFMA chain of an attention tile)
template <int SRC, int NV, int THREADS>
__global__ __launch_bounds__(THREADS) void valu_src(float* out, int iters, long long* cyc) {
  const int t = threadIdx.x, l = t & 63;
  bf16x8 a, b;
  for (int e = 0; e < 8; e++) { a[e] = (__bf16)(1.0f + l * 0.001f); b[e] = (__bf16)1.0f; }
  f32x16 c[4];
  for (int i = 0; i < 4; i++) for (int v = 0; v < 16; v++) c[i][v] = 0.f;
  float x[8];
  for (int i = 0; i < 8; i++) x[i] = l * 0.001f + i;
  long long t0 = __builtin_readcyclecounter();
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int j = 0; j < 16; j++) {
      c[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c[j & 3], 0, 0, 0);
#pragma unroll
      for (int k = 0; k < NV; k++) {
        if (SRC == 0) x[(j + k) % 8] = x[(j + k) % 8] * 0.999f + 0.5f;
        else x[(j + k) % 8] = c[(j + 2) & 3][(4 * (j >> 2) + k) & 15] * 0.999f + x[(j + k) % 8];
      }
      if (SRC == 2 && (j & 3) == 3) b[0] = (__bf16)x[j % 8];
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  long long t1 = __builtin_readcyclecounter();
  float s = 0;
  for (int i = 0; i < 4; i++) s += c[i][0];
  for (int i = 0; i < 8; i++) s += x[i];
  out[blockIdx.x * THREADS + t] = s;
  if (blockIdx.x == 0 && t == 0) cyc[0] = t1 - t0;
}

// ---- (6) does the order of the MFMAs matter for the clock the part sustains?  MFMAs alone (one wave per SIMD, every
// CU), operands from eight A and eight B fragments of normal-distributed values held in registers, long enough for
// the power management to settle.  The matrix pipe takes 32 cycles per MFMA whatever the operands, so the time of a
// fixed count is the reciprocal of the sustained clock.  REUSE 0: A and B both change with every MFMA; 1: B stays
// for four consecutive MFMAs (A changes); 2: A and B stay for four; 3: all-zero operands.
template <int REUSE>
__global__ __launch_bounds__(256) void mfma_order(const unsigned* __restrict__ src, float* out, int iters) {
  const int t = threadIdx.x, l = t & 63;
  u32x4 a[8], b[8];
  for (int i = 0; i < 8; i++) {
    a[i] = *(const u32x4*)(src + ((i * 64 + l) * 4));
    b[i] = *(const u32x4*)(src + ((512 + i * 64 + l) * 4));
    if (REUSE == 3) { a[i] = u32x4{0, 0, 0, 0}; b[i] = u32x4{0, 0, 0, 0}; }
  }
  f32x16 c[4];
  for (int i = 0; i < 4; i++) for (int v = 0; v < 16; v++) c[i][v] = 0.f;
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int j = 0; j < 32; j++) {
      const int ia = REUSE == 2 ? (j / 4) % 8 : j % 8, ib = REUSE >= 1 ? (j / 4) % 8 : (j + j / 8) % 8;
      c[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[ia]), __builtin_bit_cast(bf16x8, b[ib]), c[j & 3], 0, 0, 0);
    }
  }
  float s = 0;
  for (int i = 0; i < 4; i++) s += c[i][0];
  out[blockIdx.x * 256 + t] = s;
}

int main() {
  hipDeviceProp_t p; CK(hipGetDeviceProperties(&p, 0));
  const int ncu = p.multiProcessorCount;
  float* out; CK(hipMalloc(&out, 1024 * 512 * 4)); long long* cyc; CK(hipMalloc(&cyc, 64)); long long h[8];
  printf("CUs %d, clock %.0f MHz\n", ncu, p.clockRate / 1e3);
  {
    const int it = 4000;
#define RD(K, P, BY, name) { float ms = timeit([&] { rd<K, P><<<ncu * 2, 256>>>(out, it, cyc); }); CK(hipMemcpy(h, cyc, 8, hipMemcpyDeviceToHost)); \
    printf("%-40s %.3f ms; wave0: %.1f cycles per instruction (8 waves/CU) => %.1f B/clk/CU\n", name, ms, (double)h[0] / (it * 16.0), 8.0 * 64 * BY / ((double)h[0] / (it * 16.0))); fflush(stdout); }
    RD(0, 0, 16, "ds_read_b128 contiguous")
    RD(1, 0, 8, "ds_read_b64 contiguous")
    RD(2, 0, 8, "ds_read_b64_tr_b16 contiguous")
    RD(0, 1, 16, "ds_read_b128 fragment, swizzle row&15")
    RD(0, 2, 16, "ds_read_b128 fragment, rotated swizzle")
    RD(2, 1, 8, "ds_read_b64_tr_b16 4x64B, swizzle row&15")
    RD(2, 2, 8, "ds_read_b64_tr_b16 4x64B, rotated swizzle")
    RD(1, 2, 8, "ds_read_b64 4x64B, rotated swizzle")
  }
  {
    const int it = 2000;
#define ONE(RK, NV, NE) { float ms = timeit([&] { one<RK, NV, NE><<<ncu, 256>>>(out, it, cyc); }); CK(hipMemcpy(h, cyc, 8, hipMemcpyDeviceToHost)); \
    printf("one wave/SIMD: reads=%d valu=%d exp=%d: %.1f cycles per MFMA (%.3f ms)\n", RK, NV, NE, (double)h[0] / (it * 16.0), ms); fflush(stdout); }
    ONE(0, 0, 0) ONE(1, 0, 0) ONE(2, 0, 0) ONE(1, 2, 0) ONE(2, 2, 0) ONE(1, 3, 1) ONE(2, 3, 1) ONE(1, 4, 1) ONE(1, 6, 1) ONE(0, 3, 1) ONE(0, 6, 0) ONE(0, 8, 0)
    ONE(0, 0, 1) ONE(0, 0, 2) ONE(0, 0, 3) ONE(0, 2, 2) ONE(1, 2, 2) ONE(2, 2, 2) ONE(2, 0, 0) ONE(2, 2, 1)
  }
  {
    const int it = 500;
#define TWO(M, NM, V, E) { float ms = timeit([&] { two<M, NM, V, E><<<ncu, 512>>>(out, it, cyc); }); CK(hipMemcpy(h, cyc, 64, hipMemcpyDeviceToHost)); \
    printf("two waves/SIMD mode=%d NM=%d valu/mfma=%d exp/mfma=%d: %.1f cycles per MFMA of the SIMD (wave0 %.1f, wave4 %.1f per own MFMA) %.3f ms\n", M, NM, V, E, \
           (double)(h[0] > h[4] ? h[0] : h[4]) / (it * 2.0 * NM), (double)h[0] / (it * (double)NM), (double)h[4] / (it * (double)NM), ms); fflush(stdout); }
    TWO(0, 32, 3, 1) TWO(1, 32, 3, 1) TWO(2, 32, 3, 1) TWO(3, 32, 3, 1) TWO(4, 32, 3, 1) TWO(5, 32, 3, 1)
    TWO(0, 32, 5, 1) TWO(1, 32, 5, 1) TWO(2, 32, 5, 1) TWO(4, 32, 5, 1) TWO(5, 32, 5, 1)
    TWO(0, 16, 5, 1) TWO(2, 16, 5, 1) TWO(5, 16, 5, 1)
    TWO(0, 32, 2, 1) TWO(2, 32, 2, 1)
  }
  {
    const int it = 2000;
#define ACCK(A, CH, NV, TH) { float ms = timeit([&] { acc_kind<A, CH, NV, TH><<<ncu, TH>>>(out, it, cyc); }); CK(hipMemcpy(h, cyc, 8, hipMemcpyDeviceToHost)); \
    printf("%d wave(s)/SIMD, accumulators in %s, %d in rotation, valu/mfma=%d: %.3f ms for %d MFMAs per wave\n", TH / 256, A ? "AGPRs" : "VGPRs", CH, NV, ms, it * 16); fflush(stdout); }
    ACCK(0, 4, 0, 256) ACCK(1, 4, 0, 256) ACCK(0, 1, 0, 256) ACCK(1, 1, 0, 256)
    ACCK(0, 4, 4, 256) ACCK(1, 4, 4, 256) ACCK(0, 4, 8, 256) ACCK(1, 4, 8, 256) ACCK(0, 1, 8, 256) ACCK(1, 1, 8, 256)
    ACCK(0, 4, 0, 512) ACCK(1, 4, 0, 512)
    ACCK(0, 4, 4, 512) ACCK(1, 4, 4, 512) ACCK(0, 4, 6, 512) ACCK(1, 4, 6, 512) ACCK(0, 4, 8, 512) ACCK(1, 4, 8, 512)
    ACCK(0, 1, 6, 512) ACCK(1, 1, 6, 512)
  }
  {
    const int it = 2000;
#define VSRC(S, NV, TH) { float ms = timeit([&] { valu_src<S, NV, TH><<<ncu, TH>>>(out, it, cyc); }); \
    printf("%d wave(s)/SIMD, FMAs read %s, valu/mfma=%d: %.3f ms for %d MFMAs per wave\n", TH / 256, \
           S == 0 ? "their own registers" : S == 1 ? "an accumulator written two MFMAs earlier" : "an accumulator and feed the B operand", NV, ms, it * 16); fflush(stdout); }
    VSRC(0, 4, 256) VSRC(1, 4, 256) VSRC(2, 4, 256) VSRC(0, 4, 512) VSRC(1, 4, 512) VSRC(2, 4, 512)
    VSRC(0, 2, 256) VSRC(1, 2, 256) VSRC(0, 2, 512) VSRC(1, 2, 512) VSRC(0, 6, 512) VSRC(1, 6, 512)
  }
  {
    // normal-distributed bf16 values (Box-Muller on a fixed LCG), scaled by 1/16 so that the sums stay small
    unsigned* hsrc = (unsigned*)malloc(1024 * 4 * 4);
    unsigned long long st = 88172645463325252ull;
    auto uni = [&]() { st = st * 6364136223846793005ull + 1442695040888963407ull; return (double)((st >> 11) + 1) / 9007199254740993.0; };
    auto nbf = [&]() {
      const float f = (float)(sqrt(-2.0 * log(uni())) * cos(6.283185307179586 * uni()) / 16.0);
      unsigned u; memcpy(&u, &f, 4);
      return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    };
    for (int i = 0; i < 4096; i++) hsrc[i] = nbf() | (nbf() << 16);
    unsigned* dsrc; CK(hipMalloc(&dsrc, 4096 * 4)); CK(hipMemcpy(dsrc, hsrc, 4096 * 4, hipMemcpyHostToDevice));
    const int it = 4000;  // 128000 MFMAs per wave and launch: about 2 ms
#define ORD(R, name) { for (int w = 0; w < 150; w++) mfma_order<R><<<ncu, 256>>>(dsrc, out, it); CK(hipDeviceSynchronize()); \
    float ms = timeit([&] { for (int w = 0; w < 50; w++) mfma_order<R><<<ncu, 256>>>(dsrc, out, it); }, 3) / 50; \
    printf("MFMAs alone, %-44s %.3f ms per launch = %.0f MHz sustained\n", name, ms, 32.0 * 32 * it / (ms * 1e3)); fflush(stdout); }
    ORD(0, "A and B change with every MFMA:")
    ORD(1, "B stays for four MFMAs:")
    ORD(2, "A and B stay for four MFMAs:")
    ORD(3, "all-zero operands:")
    ORD(0, "A and B change with every MFMA (again):")
  }
  printf("done\n");
  return 0;
}
