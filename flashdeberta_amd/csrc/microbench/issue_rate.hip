// Microbenchmark for gfx950 (MI355X): how fast ONE wave issues instructions, by kind, alone on its SIMD and with a
// second wave beside it.  The near kernel of this library runs two waves per SIMD, and a 32-key step of it is a few
// hundred instructions of every kind (vector, scalar, LDS, waits) around twenty MFMAs: whether the step is bound
// by a unit or by the wave's own issue rate decides what is worth removing from it.
//
//   hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         flashdeberta_amd/csrc/microbench/issue_rate.hip -o issue_rate && ./issue_rate
//
// Every loop body is inline asm (exact instruction order, independent instructions, no memory traffic); times are
// s_memtime differences inside the kernel (core clocks) of the first wave of workgroup 0, per instruction.
// Workgroups of 256 threads (one wave per SIMD); the launch asks for as much LDS as leaves room for exactly one or
// two workgroups per CU.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define CHECK(x)                                                            \
  do {                                                                      \
    hipError_t e_ = (x);                                                    \
    if (e_ != hipSuccess) {                                                 \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      return 1;                                                             \
    }                                                                       \
  } while (0)

#define REP4(x) x x x x
#define REP16(x) REP4(x) REP4(x) REP4(x) REP4(x)

// 64 instructions per iteration
template <int KIND>
__global__ __launch_bounds__(256) void issue_kernel(unsigned long long* out, int iters) {
  extern __shared__ char smem[];
  float a = threadIdx.x, b = 1.f, c = 2.f, d = 3.f;
  unsigned long long t0, t1;
  asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t0)::"memory");
  for (int it = 0; it < iters; ++it) {
    if (KIND == 0) {  // vector: independent v_fma_f32 on four registers
      asm volatile(REP16("v_fma_f32 %0, %0, %0, %0\n\tv_fma_f32 %1, %1, %1, %1\n\tv_fma_f32 %2, %2, %2, %2\n\tv_fma_f32 %3, %3, %3, %3\n\t")
                   : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    } else if (KIND == 1) {  // scalar
      asm volatile(REP16("s_add_u32 s40, s40, 1\n\ts_add_u32 s41, s41, 1\n\ts_add_u32 s42, s42, 1\n\ts_add_u32 s43, s43, 1\n\t") ::
                       : "s40", "s41", "s42", "s43", "scc");
    } else if (KIND == 2) {  // vector and scalar alternating
      asm volatile(REP16("v_fma_f32 %0, %0, %0, %0\n\ts_add_u32 s40, s40, 1\n\tv_fma_f32 %1, %1, %1, %1\n\ts_add_u32 s41, s41, 1\n\t")
                   : "+v"(a), "+v"(b)
                   :
                   : "s40", "s41", "scc");
    } else if (KIND == 3) {  // lane rotations through the LDS pipe (no memory), results never waited for inside the block
      asm volatile(REP16("ds_swizzle_b32 %0, %0 offset:0xC020\n\tds_swizzle_b32 %1, %1 offset:0xC040\n\tds_swizzle_b32 %2, %2 offset:0xC060\n\t"
                         "ds_swizzle_b32 %3, %3 offset:0xC080\n\t") "s_waitcnt lgkmcnt(0)\n\t"
                   : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    } else if (KIND == 4) {  // vector, scalar, rotation and a satisfied wait in turn: the mix of an attention step
      asm volatile(REP16("v_fma_f32 %0, %0, %0, %0\n\ts_add_u32 s40, s40, 1\n\tds_swizzle_b32 %1, %1 offset:0xC020\n\ts_waitcnt vmcnt(0)\n\t")
                       "s_waitcnt lgkmcnt(0)\n\t"
                   : "+v"(a), "+v"(b)
                   :
                   : "s40", "scc");
    } else if (KIND == 5) {  // waits that are already satisfied and nops
      asm volatile(REP16("s_waitcnt vmcnt(0)\n\ts_nop 0\n\ts_waitcnt lgkmcnt(0)\n\ts_nop 0\n\t") ::: "memory");
    } else if (KIND == 6) {  // the exponential of the soft-max (transcendental unit)
      asm volatile(REP16("v_exp_f32 %0, %0\n\tv_exp_f32 %1, %1\n\tv_exp_f32 %2, %2\n\tv_exp_f32 %3, %3\n\t")
                   : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    } else if (KIND == 7) {  // exponentials and plain vector instructions in turn, as in the soft-max of a key tile (2 : 3)
      asm volatile(REP16("v_exp_f32 %0, %0\n\tv_add_f32 %2, %2, %3\n\tv_exp_f32 %1, %1\n\tv_add_f32 %3, %3, %2\n\t")
                   : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    } else if (KIND == 8) {  // conversion of two fp32 values to packed bf16
      asm volatile(REP16("v_cvt_pk_bf16_f32 %0, %0, %1\n\tv_cvt_pk_bf16_f32 %1, %1, %2\n\tv_cvt_pk_bf16_f32 %2, %2, %3\n\tv_cvt_pk_bf16_f32 %3, %3, %0\n\t")
                   : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    } else {  // arbitrary lane permutation through the LDS pipe (address register per lane)
      asm volatile(REP16("ds_bpermute_b32 %0, %1, %0\n\tds_bpermute_b32 %2, %1, %2\n\tds_bpermute_b32 %3, %1, %3\n\t"
                         "ds_bpermute_b32 %0, %1, %0\n\t") "s_waitcnt lgkmcnt(0)\n\t"
                   : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    }
  }
  asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t1)::"memory");
  if (blockIdx.x == 0 && threadIdx.x == 0) out[0] = t1 - t0;
  if (a + b + c + d == 12345.f) out[1] = 1;
}

static int g_cus = 256;
static int lds_for(int per_cu) { return (160 * 1024) / per_cu - 1024; }

template <int KIND>
int run(const char* name, unsigned long long* d) {
  const int iters = 2000;
  double per[2];
  for (int wps = 1; wps <= 2; ++wps) {
    auto kern = issue_kernel<KIND>;
    const int lds = lds_for(wps);
    CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    for (int rep = 0; rep < 2; ++rep) {
      hipLaunchKernelGGL(kern, dim3(g_cus * wps), dim3(256), lds, 0, d, iters);
      CHECK(hipDeviceSynchronize());
    }
    unsigned long long h = 0;
    CHECK(hipMemcpy(&h, d, 8, hipMemcpyDeviceToHost));
    per[wps - 1] = (double)h / iters / 64.0;
  }
  printf("%-58s %5.2f clocks per instruction alone, %5.2f with a second wave of the same kind on the SIMD\n", name, per[0], per[1]);
  return 0;
}

int main() {
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  g_cus = prop.multiProcessorCount;
  printf("%s, %d CUs\n", prop.gcnArchName, g_cus);
  unsigned long long* d;
  CHECK(hipMalloc(&d, 64));
  CHECK(hipMemset(d, 0, 64));
  return run<0>("v_fma_f32 (independent)", d) || run<1>("s_add_u32 (independent)", d) || run<2>("v_fma_f32 / s_add_u32 alternating", d) ||
         run<3>("ds_swizzle_b32 (lane rotation, LDS pipe)", d) || run<4>("v_fma_f32 / s_add_u32 / ds_swizzle_b32 / satisfied s_waitcnt", d) ||
         run<5>("satisfied s_waitcnt / s_nop 0", d) || run<6>("v_exp_f32 (independent)", d) || run<7>("v_exp_f32 / v_add_f32 alternating", d) ||
         run<8>("v_cvt_pk_bf16_f32", d) || run<9>("ds_bpermute_b32 (lane permutation, LDS pipe)", d);
}
