// Microbenchmark for gfx950 (MI355X): how matrix (MFMA) and vector (VALU) instructions share a SIMD, and what
// that leaves of the MFMA peak for an attention tile.  The attention kernels of this library alternate MFMA phases
// (scores, P V) with VALU phases (exponentials, conversions, row sums); whether the two kinds of work overlap, and
// at what clock, decides what fraction of the 2.5 PFLOP/s such a kernel can reach before it touches memory.
//
//   hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         flashdeberta_amd/csrc/microbench/issue_overlap.hip -o issue_overlap && ./issue_overlap
//
// No memory traffic anywhere.  Every launch asks for as much LDS as leaves room for exactly the intended number of
// workgroups per CU (the dispatcher would otherwise be free to put more of them on some CUs and none on others).
// Times are HIP-event times of the whole launch (the best of three), converted to cycles at the nominal 2.4 GHz; "core clocks" are s_memtime differences inside the kernel, so the ratio of the two
// is the clock the GPU actually ran at.
//   A  issue rate of independent MFMAs: bf16 32x32x16, e4m3 32x32x16, e4m3 32x32x64
//   B  one wave per SIMD, exact instruction order (inline asm): 1 MFMA followed by N independent v_fma_f32
//   C  two waves per SIMD (paired by hardware SIMD id), one issuing only MFMAs, the other only VALU instructions,
//      with and without a higher priority for the VALU wave
//   D  a far tile of the attention kernels (8 MFMAs of scores, 32 exponentials + 16 conversions + 32 adds, 8 MFMAs
//      of P V): 1 to 4 independent waves per SIMD; two waves per SIMD half a tile apart, with and without workgroup
//      barriers between the phases; three waves per SIMD one phase apart with a barrier after every phase
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

typedef __attribute__((ext_vector_type(8))) int v8i;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(16))) float v16f;
typedef __attribute__((ext_vector_type(4))) int v4i;

#define CHECK(x)                                                                     \
  do {                                                                               \
    hipError_t e_ = (x);                                                             \
    if (e_ != hipSuccess) {                                                          \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);          \
      return 1;                                                                      \
    }                                                                                \
  } while (0)

static int g_cus = 256;
// dynamic LDS that lets exactly `per_cu` workgroups share a CU's 160 KB
static int lds_for(int per_cu) { return 160 * 1024 / per_cu - 1024; }

// best-of-three event time of one launch, in ms
template <class F>
static int timed(F launch, float* ms_out) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  float best = 1e30f;
  for (int rep = 0; rep < 3; ++rep) {
    CHECK(hipEventRecord(e0));
    launch();
    CHECK(hipEventRecord(e1));
    CHECK(hipDeviceSynchronize());
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    if (ms < best) best = ms;
  }
  *ms_out = best;
  return 0;
}

// ---- A ------------------------------------------------------------------------------------------------------
template <int MODE>
__global__ __launch_bounds__(256) void rate_kernel(float* out, int iters) {
  v16f c0 = {}, c1 = {}, c2 = {}, c3 = {};
  const int t = threadIdx.x;
  v8i a8 = {t, t + 1, t + 2, t + 3, t + 4, t + 5, t + 6, t + 7}, b8 = {t * 3, 1, 2, 3, 4, 5, 6, 7};
  bf16x8 ab = __builtin_bit_cast(bf16x8, v4i{t, 1, 2, 3});
  bf16x8 bb = __builtin_bit_cast(bf16x8, v4i{t * 5, 1, 2, 3});
  long al = t * 77, bl = t * 91;
  for (int i = 0; i < iters; ++i) {
    if (MODE == 0) {
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ab, bb, c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ab, bb, c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ab, bb, c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ab, bb, c3, 0, 0, 0);
    } else if (MODE == 1) {
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(al, bl, c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(al, bl, c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(al, bl, c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(al, bl, c3, 0, 0, 0);
    } else {
      c0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c0, 0, 0, 0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c1, 0, 0, 0, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c2, 0, 0, 0, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c3, 0, 0, 0, 0, 0, 0);
    }
  }
  v16f s = c0 + c1 + c2 + c3;
  float r = 0;
  for (int e = 0; e < 16; ++e) r += s[e];
  out[blockIdx.x * 256 + t] = r;
}

template <int MODE>
static int run_rate(const char* name, float* d, int k_per, int wgs_per_cu) {
  const int iters = 20000;
  float ms;
  CHECK(hipFuncSetAttribute((const void*)rate_kernel<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_for(1)));
  if (timed([&] { rate_kernel<MODE><<<g_cus * wgs_per_cu, 256, lds_for(wgs_per_cu)>>>(d, iters); }, &ms)) return 1;
  const double mfma_per_simd = (double)iters * 4 * wgs_per_cu;
  const double flop = mfma_per_simd * 4.0 * g_cus * 32 * 32 * k_per * 2;
  printf("A  %-24s %d wave(s)/SIMD: %6.1f cycles per MFMA per SIMD, %7.1f TFLOP/s\n", name, wgs_per_cu,
         ms * 1e6 * 2.4 / mfma_per_simd, flop / (ms * 1e-3) / 1e12);
  return 0;
}

// ---- B ------------------------------------------------------------------------------------------------------
template <int N>
__global__ __launch_bounds__(256, 1) void serial_kernel(float* out, int iters) {
  v16f c = {};
  const int t = threadIdx.x;
  bf16x8 a = __builtin_bit_cast(bf16x8, v4i{t, 1, 2, 3}), b = __builtin_bit_cast(bf16x8, v4i{t * 5, 1, 2, 3});
  float x[12];
  for (int e = 0; e < 12; ++e) x[e] = 0.001f * (t + e);
  const float m = 0.999f, q = 0.0001f;
  for (int i = 0; i < iters; ++i) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
#pragma unroll
    for (int e = 0; e < N; ++e) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[e]) : "v"(m), "v"(q));
  }
  float r = 0;
  for (int e = 0; e < 16; ++e) r += c[e];
  for (int e = 0; e < 12; ++e) r += x[e];
  out[blockIdx.x * 256 + t] = r;
}
template <int N>
static int run_serial(float* d, double* cycles) {
  const int iters = 100000;
  float ms;
  CHECK(hipFuncSetAttribute((const void*)serial_kernel<N>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_for(1)));
  if (timed([&] { serial_kernel<N><<<g_cus, 256, lds_for(1)>>>(d, iters); }, &ms)) return 1;
  *cycles = ms * 1e6 * 2.4 / iters;
  return 0;
}

// ---- pairing two waves on one SIMD ---------------------------------------------------------------------------
// A 512-thread workgroup has two waves on each SIMD, but which two is the dispatcher's business: every wave reads
// its SIMD id and the first to arrive on a SIMD takes role 0, the second role 1.
__device__ __forceinline__ int take_role(int* cnt) {
  unsigned id;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(id));
  const int simd = (id >> 4) & 3;
  int role = 0;
  if ((threadIdx.x & 63) == 0) role = atomicAdd(&cnt[simd], 1);
  return __builtin_amdgcn_readfirstlane(role);
}

__device__ long long g_clk[2];
__device__ long long g_wave_clk[8192];  // per wave: core clocks spent in the loop

// ---- C ------------------------------------------------------------------------------------------------------
// role 0: na x [16 MFMAs on two accumulator chains]; role 1: nb x [the VALU phase of a tile on loop-carried data]
__device__ __forceinline__ void valu_phase(const v16f& s0, const v16f& s1, bf16x8 (&p)[4], float& l) {
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    f32x8 pv;
#pragma unroll
    for (int e = 0; e < 8; ++e) pv[e] = __builtin_amdgcn_exp2f((c < 2 ? s0 : s1)[8 * (c & 1) + e]);
    p[c] = __builtin_convertvector(pv, bf16x8);
    l += ((pv[0] + pv[1]) + (pv[2] + pv[3])) + ((pv[4] + pv[5]) + (pv[6] + pv[7]));
  }
}
template <int PRIO>
__global__ __launch_bounds__(512, 1) void pair_kernel(float* out, int na, int nb) {
  __shared__ int cnt[4];
  const int t = threadIdx.x;
  if (t < 4) cnt[t] = 0;
  __syncthreads();
  const int role = take_role(cnt);
  __syncthreads();
  if (PRIO) {
    if (role == 1) __builtin_amdgcn_s_setprio(3);
    else __builtin_amdgcn_s_setprio(0);
  }
  float r = 0;
  const long long t0 = clock64();
  if (role == 0) {
    v16f c0 = {}, c1 = {};
    bf16x8 a = __builtin_bit_cast(bf16x8, v4i{t, 1, 2, 3}), b = __builtin_bit_cast(bf16x8, v4i{t * 5, 1, 2, 3});
    for (int i = 0; i < na; ++i) {
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
      }
    }
    for (int e = 0; e < 16; ++e) r += c0[e] + c1[e];
  } else {
    v16f s0, s1;
    for (int e = 0; e < 16; ++e) {
      s0[e] = -0.001f * (t + e);
      s1[e] = -0.002f * (t + e);
    }
    float l = 0.f;
    bf16x8 p[4];
    for (int i = 0; i < nb; ++i) {
      valu_phase(s0, s1, p, l);
#pragma unroll
      for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(p[c]));
      asm volatile("" : "+v"(s0), "+v"(s1));
    }
    r = l;
    for (int c = 0; c < 4; ++c) r += (float)p[c][0];
  }
  const long long t1 = clock64();
  out[blockIdx.x * 512 + t] = r;
  if ((t & 63) == 0 && blockIdx.x == 33) g_clk[role] = t1 - t0;
}
template <int PRIO>
static int run_pair(const char* name, float* d) {
  const int n = 20000;
  float ms[3];
  long long clk[3][2];
  CHECK(hipFuncSetAttribute((const void*)pair_kernel<PRIO>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_for(1)));
  for (int mode = 0; mode < 3; ++mode) {
    if (timed([&] { pair_kernel<PRIO><<<g_cus, 512, lds_for(1)>>>(d, mode == 1 ? 0 : n, mode == 0 ? 0 : n); }, &ms[mode])) return 1;
    CHECK(hipMemcpyFromSymbol(clk[mode], HIP_SYMBOL(g_clk), sizeof clk[mode]));
  }
  const double c24 = 1e6 * 2.4 / n;
  printf("C  %-34s MFMA wave alone %6.1f, VALU wave alone %6.1f, both on one SIMD %6.1f cycles@2.4GHz per iteration\n"
         "   %-34s core clocks per iteration with both: MFMA wave %.0f, VALU wave %.0f  => clock %.2f GHz (alone: %.2f / %.2f)\n",
         name, ms[0] * c24, ms[1] * c24, ms[2] * c24, "", (double)clk[2][0] / n, (double)clk[2][1] / n,
         (double)clk[2][1] / n / (ms[2] * 1e6 / n), (double)clk[0][0] / n / (ms[0] * 1e6 / n), (double)clk[1][1] / n / (ms[1] * 1e6 / n));
  return 0;
}

// ---- D ------------------------------------------------------------------------------------------------------
// MODE 0: 256-thread workgroups, WPS per CU, every wave runs scores -> VALU phase -> P V one after the other;
// MODE 1: one 512-thread workgroup per CU, the second wave of every SIMD half a tile behind the first, workgroup
//         barriers between the phases (explicit ping-pong: between two barriers one wave of a SIMD issues only MFMAs,
//         the other only VALU instructions);  MODE 2: the same offset at the start and no barriers afterwards;
// MODE 3: one 768-thread workgroup per CU, three waves per SIMD one phase apart (scores | VALU phase | P V), a workgroup
//         barrier after every phase: at any time one wave of a SIMD is in each of the three phases.
template <int MODE, int WPS>
__global__ __launch_bounds__(MODE == 3 ? 768 : MODE ? 512 : 256, MODE ? 1 : WPS) void tile_kernel(float* out, int iters, float seed) {
  __shared__ int cnt[4];
  int role = 0;
  if (MODE) {
    if (threadIdx.x < 4) cnt[threadIdx.x] = 0;
    __syncthreads();
    role = take_role(cnt);
    __syncthreads();
  }
  bf16x8 a[4], b[4];
  for (int i = 0; i < 4; ++i)
    for (int e = 0; e < 8; ++e) {
      a[i][e] = (__bf16)(seed * (threadIdx.x + i + e));
      b[i][e] = (__bf16)(seed * (threadIdx.x * 3 + i - e));
    }
  v16f o0 = {}, o1 = {}, s0 = {}, s1 = {};
  bf16x8 p[4] = {a[0], a[1], a[2], a[3]};
  float l = 0.f;
  auto scores = [&]() __attribute__((always_inline)) {
    v16f z = {};
    s0 = z;
    s1 = z;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[x], b[x], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[x], a[x], s1, 0, 0, 0);
    }
  };
  auto pv = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      o0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[c], p[c], o0, 0, 0, 0);
      o1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[c], p[c], o1, 0, 0, 0);
    }
  };
  const long long t0 = clock64();
  if (MODE == 0) {
    for (int it = 0; it < iters; ++it) {
      scores();
      __builtin_amdgcn_sched_barrier(0);
      valu_phase(s0, s1, p, l);
      __builtin_amdgcn_sched_barrier(0);
      pv();
      __builtin_amdgcn_sched_barrier(0);
    }
  } else if (MODE == 3) {
    for (int e = 0; e < role; ++e) __syncthreads();
    for (int it = 0; it < iters; ++it) {
      scores();
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
      valu_phase(s0, s1, p, l);
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
      pv();
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
    }
    for (int e = role; e < 2; ++e) __syncthreads();
  } else {
    scores();
    if (role == 1) {
      if (MODE == 1) __syncthreads();
      else __builtin_amdgcn_s_sleep(8);
    }
    for (int it = 0; it < iters; ++it) {
      __builtin_amdgcn_sched_barrier(0);
      valu_phase(s0, s1, p, l);
      __builtin_amdgcn_sched_barrier(0);
      if (MODE == 1) __syncthreads();
      pv();
      scores();
      __builtin_amdgcn_sched_barrier(0);
      if (MODE == 1) __syncthreads();
    }
    if (role == 0 && MODE == 1) __syncthreads();
  }
  const long long t1 = clock64();
  float acc = l;
  for (int v = 0; v < 16; ++v) acc += o0[v] + o1[v] + s0[v] + s1[v];
  out[blockIdx.x * 512 + threadIdx.x] = acc;
  if ((threadIdx.x & 63) == 0) g_wave_clk[blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)] = t1 - t0;
}
template <int MODE, int WPS>
static int run_tile(const char* name, float* d) {
  const int iters = 20000;
  float ms;
  CHECK(hipFuncSetAttribute((const void*)tile_kernel<MODE, WPS>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_for(1)));
  if (timed([&] { tile_kernel<MODE, WPS><<<g_cus * (MODE ? 1 : WPS), MODE == 3 ? 768 : MODE ? 512 : 256, lds_for(MODE ? 1 : WPS)>>>(d, iters, 0.001f); }, &ms)) return 1;
  static long long clk[8192];
  CHECK(hipMemcpyFromSymbol(clk, HIP_SYMBOL(g_wave_clk), sizeof clk));
  const int waves_per_simd = MODE == 3 ? 3 : MODE ? 2 : WPS, waves = g_cus * 4 * waves_per_simd;
  double hi = 0, mean = 0;
  for (int i = 0; i < waves; ++i) {
    hi = clk[i] > hi ? (double)clk[i] : hi;
    mean += (double)clk[i] / waves;
  }
  // a wave runs `iters` tiles; a SIMD runs waves_per_simd of them side by side
  const double per_tile = ms * 1e6 * 2.4 / iters / waves_per_simd;
  printf("D  %-62s %6.1f cycles@2.4GHz per tile and SIMD = %4.1f %% of the MFMA peak\n"
         "   %-62s core clocks per tile of a wave: mean %.0f, slowest %.0f; clock of the slowest wave %.2f GHz\n", name,
         per_tile, 100.0 * 512.0 / per_tile, "", mean / iters, hi / iters, hi / (ms * 1e6));
  return 0;
}

int main() {
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  g_cus = prop.multiProcessorCount;
  printf("%s, %d CUs\n", prop.gcnArchName, g_cus);
  float* d;
  CHECK(hipMalloc(&d, 4 * 512 * 4 * 1024));
  for (int w = 1; w <= 4; w *= 2)
    if (run_rate<0>("bf16 32x32x16", d, 16, w) || run_rate<1>("e4m3 32x32x16", d, 16, w) || run_rate<2>("e4m3 32x32x64 (f8f6f4)", d, 64, w))
      return 1;
  double c[7];
  if (run_serial<0>(d, &c[0]) || run_serial<2>(d, &c[1]) || run_serial<4>(d, &c[2]) || run_serial<6>(d, &c[3]) ||
      run_serial<8>(d, &c[4]) || run_serial<10>(d, &c[5]) || run_serial<12>(d, &c[6]))
    return 1;
  printf("B  one wave per SIMD, [1 dependent MFMA 32x32x16, N independent v_fma_f32] per iteration\n   N =        0      2      4      6      8     10     12\n   cycles");
  for (int i = 0; i < 7; ++i) printf(" %6.1f", c[i]);
  printf("\n");
  if (run_pair<0>("two waves, equal priority:", d) || run_pair<1>("two waves, VALU wave prioritised:", d)) return 1;
  if (run_tile<0, 1>("tile loop, one wave per SIMD", d) || run_tile<0, 2>("tile loop, two independent waves per SIMD", d) ||
      run_tile<0, 3>("tile loop, three independent waves per SIMD", d) || run_tile<0, 4>("tile loop, four independent waves per SIMD", d) ||
      run_tile<1, 1>("tile loop, two waves per SIMD half a tile apart, barriers", d) ||
      run_tile<2, 1>("tile loop, two waves per SIMD half a tile apart, free-running", d) ||
      run_tile<3, 1>("tile loop, three waves per SIMD a phase apart, barriers", d))
    return 1;
  return 0;
}
