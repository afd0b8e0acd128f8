// Device-side building blocks shared by the attention kernels: vector typedefs, element traits
// (MFMA operand fragments per dtype), the V^T operand loader and the half-wave exchange.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define LDS_AS __attribute__((address_space(3)))

namespace fdb {

constexpr float kLazyTau = 8.f;  // the running reference point of a row is moved only when the tile
                                 // maximum exceeds it by more than 2^8 (any reference point is valid)

// ---- element traits --------------------------------------------------------------------------
// frag: the 8 contraction elements one lane feeds to a K=16 step (lane = outer index l%32, the
// elements are k = 16*step + 8*(l/32) + 0..7).
struct Bf16Tr {
  static constexpr int SZ = 2;
  static constexpr uint32_t NAN_WORD = 0x7FC07FC0u;  // a quiet NaN in every element of a 32-bit word
  using frag = bf16x8;
  using scratch_t = __bf16;
  static __device__ __forceinline__ frag zero() { return frag{0, 0, 0, 0, 0, 0, 0, 0}; }
  static __device__ __forceinline__ frag load(const void* p) { return *(const frag*)p; }
  static __device__ __forceinline__ f32x16 mma(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x8 to_f32(frag x) { return __builtin_convertvector(x, f32x8); }
  static __device__ __forceinline__ frag from_f32(f32x8 x) { return __builtin_convertvector(x, frag); }
  static __device__ __forceinline__ void store4(char* p, float a, float b, float c, float d) {
    f32x4 x = {a, b, c, d};
    *(bf16x4*)p = __builtin_convertvector(x, bf16x4);
  }
  // acc + the low / high element of a packed pair, one instruction each.  The selectors carry -0
  // in the unused half: (1, +0) would be encoded as the inline constant 1.0, which the dot
  // instruction reads as the fp32 pattern, i.e. as (+0, 1).
  static __device__ __forceinline__ float add_lo(float acc, uint32_t pair) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pair), bf16x2{(__bf16)1.0f, (__bf16)-0.0f}, acc, false);
  }
  static __device__ __forceinline__ float add_hi(float acc, uint32_t pair) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pair), bf16x2{(__bf16)-0.0f, (__bf16)1.0f}, acc, false);
  }
  static __device__ __forceinline__ f32x4 load4(const char* p) { return __builtin_convertvector(*(const bf16x4*)p, f32x4); }
  // four fp32 values rounded to the type, and one 16-bit pattern of the type back as fp32
  using scratch4 = bf16x4;
  static __device__ __forceinline__ scratch4 pack4(f32x4 x) { return __builtin_convertvector(x, bf16x4); }
  static __device__ __forceinline__ float scratch_to_f32(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
};

struct F16Tr {
  static constexpr int SZ = 2;
  static constexpr uint32_t NAN_WORD = 0x7E007E00u;
  using frag = f16x8;
  using scratch_t = _Float16;
  static __device__ __forceinline__ frag zero() { return frag{0, 0, 0, 0, 0, 0, 0, 0}; }
  static __device__ __forceinline__ frag load(const void* p) { return *(const frag*)p; }
  static __device__ __forceinline__ f32x16 mma(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x8 to_f32(frag x) { return __builtin_convertvector(x, f32x8); }
  static __device__ __forceinline__ frag from_f32(f32x8 x) { return __builtin_convertvector(x, frag); }
  static __device__ __forceinline__ void store4(char* p, float a, float b, float c, float d) {
    f32x4 x = {a, b, c, d};
    *(f16x4*)p = __builtin_convertvector(x, f16x4);
  }
  static __device__ __forceinline__ float add_lo(float acc, uint32_t pair) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pair), f16x2{(_Float16)1.0f, (_Float16)-0.0f}, acc, false);
  }
  static __device__ __forceinline__ float add_hi(float acc, uint32_t pair) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pair), f16x2{(_Float16)-0.0f, (_Float16)1.0f}, acc, false);
  }
  static __device__ __forceinline__ f32x4 load4(const char* p) { return __builtin_convertvector(*(const f16x4*)p, f32x4); }
  using scratch4 = f16x4;
  static __device__ __forceinline__ scratch4 pack4(f32x4 x) { return __builtin_convertvector(x, f16x4); }
  static __device__ __forceinline__ float scratch_to_f32(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
};

struct F32Tr {
  static constexpr int SZ = 4;
  static constexpr uint32_t NAN_WORD = 0x7FC00000u;
  using frag = f32x8;
  using scratch_t = float;
  static __device__ __forceinline__ frag zero() { return frag{0, 0, 0, 0, 0, 0, 0, 0}; }
  static __device__ __forceinline__ frag load(const void* p) { return *(const frag*)p; }
  // A K=16 step in fp32 is eight K=2 MFMAs; lane group g supplies k = 16*step + 8*g + e to the e-th.
  static __device__ __forceinline__ f32x16 mma(frag a, frag b, f32x16 c) {
#pragma unroll
    for (int e = 0; e < 8; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
    return c;
  }
  static __device__ __forceinline__ f32x8 to_f32(frag x) { return x; }
  static __device__ __forceinline__ frag from_f32(f32x8 x) { return x; }
  static __device__ __forceinline__ void store4(char* p, float a, float b, float c, float d) {
    *(f32x4*)p = f32x4{a, b, c, d};
  }
  static __device__ __forceinline__ f32x4 load4(const char* p) { return *(const f32x4*)p; }
  static __device__ __forceinline__ float add_lo(float acc, uint32_t) { return acc; }  // 16-bit scratch only
  static __device__ __forceinline__ float add_hi(float acc, uint32_t) { return acc; }
};

struct Fp8Tr {  // OCP e4m3, operands of the three score products only
  static constexpr int SZ = 1;
  using frag = long;
  using scratch_t = __bf16;
  static __device__ __forceinline__ frag zero() { return 0; }
  static __device__ __forceinline__ frag load(const void* p) { return *(const long*)p; }
  static __device__ __forceinline__ f32x16 mma(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x8 to_f32(frag) { return f32x8{0, 0, 0, 0, 0, 0, 0, 0}; }  // unused
  static __device__ __forceinline__ frag from_f32(f32x8) { return 0; }                             // unused
  static __device__ __forceinline__ float add_lo(float acc, uint32_t) { return acc; }               // unused
  static __device__ __forceinline__ float add_hi(float acc, uint32_t) { return acc; }
};

// Row-sum contribution of eight probabilities, in fp32 and before they are rounded for the MFMA: plain
// adds.  (A 16-bit dot product per pair would halve the instruction count, but the dot instructions do not
// run beside MFMAs of other waves, and a key tile is short of exactly that overlap: 2.5 % of the far launch.)
__device__ __forceinline__ float sum8(const f32x8& x, float acc) {
  return acc + (((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7])));
}

// V^T operand of a K=16 step: lane (d = l%32, g = l/32) needs V[j(g,e)][d] for
// j(g,e) = 16*c + 8*(e/4) + 4*g + e%4 -- the key rows whose probabilities sit in this lane
// group's accumulator registers.  V stays row-major in LDS.
template <class VT>
struct VtLoad;

template <>
struct VtLoad<F32Tr> {
  static __device__ __forceinline__ f32x8 get(const char* vs, int rs, int c, int db, int lane) {
    const int li = lane & 31, g = lane >> 5;
    f32x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int row = 16 * c + 8 * (e >> 2) + 4 * g + (e & 3);
      r[e] = *(const float*)(vs + row * rs + (db * 32 + li) * 4);
    }
    return r;
  }
};

// 16-bit: ds_read_tr16_b64.  Within each group of 16 lanes, source lane s supplies an 8-byte
// address; destination lane i receives element (i%4) of source lanes 4*r + i/4, r = 0..3.
// With source lane s pointing at V[row0 + s/4][col0 + 4*(s%4) ..+3], lane i gets column
// col0 + i of rows row0 .. row0+3.
template <class VT>
struct VtLoad16 {
  static __device__ __forceinline__ typename VT::frag get(const char* vs, int rs, int c, int db, int lane) {
    const int s = lane & 15, grp = lane >> 4;
    const int row = 16 * c + 4 * (grp >> 1) + (s >> 2);
    const int col = db * 32 + 16 * (grp & 1) + 4 * (s & 3);
    const char* a = vs + row * rs + col * 2;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(a));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(a + 8 * rs));
    s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(typename VT::frag, both);
  }
};
template <>
struct VtLoad<Bf16Tr> : VtLoad16<Bf16Tr> {};
template <>
struct VtLoad<F16Tr> : VtLoad16<F16Tr> {};

// combine lane l with lane l^32 (the other half of the row's keys)
// v_permlane32_swap exchanges lanes 32..63 of its first operand with lanes 0..31 of its second.
// Fed two registers holding the same value, every lane ends up with its own value in one register
// and its partner's (lane ^ 32) in the other.  Written as one asm block: the two operands must be
// distinct registers, and the results must stay opaque to the optimiser.
__device__ __forceinline__ void half_pair(float x, float& r0, float& r1) {
  float a = x, b;
  asm volatile("v_mov_b32 %1, %0\n\ts_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "=&v"(b));
  r0 = a;
  r1 = b;
}
__device__ __forceinline__ float wave_half_max(float x) {
  float a, b;
  half_pair(x, a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float wave_half_sum(float x) {
  float a, b;
  half_pair(x, a, b);
  return a + b;
}


template <class ST>
__device__ __forceinline__ void store4_scratch(ST* p, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void store4_scratch<float>(float* p, float a, float b, float c, float d) {
  *(f32x4*)p = f32x4{a, b, c, d};
}
template <>
__device__ __forceinline__ void store4_scratch<__bf16>(__bf16* p, float a, float b, float c, float d) {
  f32x4 x = {a, b, c, d};
  *(bf16x4*)p = __builtin_convertvector(x, bf16x4);
}
template <>
__device__ __forceinline__ void store4_scratch<_Float16>(_Float16* p, float a, float b, float c, float d) {
  f32x4 x = {a, b, c, d};
  *(f16x4*)p = __builtin_convertvector(x, f16x4);
}

// Four consecutive scratch elements from an address aligned only to the element size (gfx950
// serves unaligned DS accesses), as fp32.
template <class ST>
__device__ __forceinline__ f32x4 load4_scratch_unaligned(const ST* p);
template <>
__device__ __forceinline__ f32x4 load4_scratch_unaligned<float>(const float* p) {
  typedef f32x4 __attribute__((aligned(4))) f32x4_u;
  return *(const f32x4_u*)p;
}
template <>
__device__ __forceinline__ f32x4 load4_scratch_unaligned<__bf16>(const __bf16* p) {
  typedef bf16x4 __attribute__((aligned(2))) bf16x4_u;
  return __builtin_convertvector(*(const bf16x4_u*)p, f32x4);
}
template <>
__device__ __forceinline__ f32x4 load4_scratch_unaligned<_Float16>(const _Float16* p) {
  typedef f16x4 __attribute__((aligned(2))) f16x4_u;
  return __builtin_convertvector(*(const f16x4_u*)p, f32x4);
}

// acc + the low / high element of a packed pair of 16-bit scratch values
template <class ST>
__device__ __forceinline__ float scratch_add_lo(float acc, uint32_t pair);
template <class ST>
__device__ __forceinline__ float scratch_add_hi(float acc, uint32_t pair);
template <>
__device__ __forceinline__ float scratch_add_lo<__bf16>(float acc, uint32_t pair) { return Bf16Tr::add_lo(acc, pair); }
template <>
__device__ __forceinline__ float scratch_add_hi<__bf16>(float acc, uint32_t pair) { return Bf16Tr::add_hi(acc, pair); }
template <>
__device__ __forceinline__ float scratch_add_lo<_Float16>(float acc, uint32_t pair) { return F16Tr::add_lo(acc, pair); }
template <>
__device__ __forceinline__ float scratch_add_hi<_Float16>(float acc, uint32_t pair) { return F16Tr::add_hi(acc, pair); }
template <>
__device__ __forceinline__ float scratch_add_lo<float>(float acc, uint32_t) { return acc; }  // fp32 scratch is read element-wise
template <>
__device__ __forceinline__ float scratch_add_hi<float>(float acc, uint32_t) { return acc; }

// Linear workgroup id -> (query-tile index within the launch, head).  The hardware deals
// workgroups to the 8 XCDs round-robin by linear id, and each XCD has its own L2.  In the fixed
// layout, when the number of (sequence, head) groups is a multiple of 8, groups are dealt to XCDs
// whole: all query tiles of a group then stream the same K and V through one L2.
// Within a group the query tiles are dealt in the order `order` asks for, so that the workgroups
// with the most key tiles start first and the launch ends on the short ones: kEdgesFirst for the far
// tiles (a query tile at either end of the sequence has the most), kMiddleFirst for the near tiles, kLastFirst for
// the far tiles of a causal call (a query tile sees the keys before it: the last one has the most).
enum { kNatural = 0, kEdgesFirst = 1, kMiddleFirst = 2, kLastFirst = 3 };
__device__ __forceinline__ void block_map(int n, int nx, int heads, int tiles_per_seq, bool fixed, int order, int& xq,
                                          int& h) {
  const int groups = fixed ? (nx / tiles_per_seq) * heads : 1;
  if (fixed && (groups & 7) == 0) {
    const int xcd = n & 7, slot = n >> 3;
    const int grp = xcd + 8 * (slot / tiles_per_seq);
    int t = slot % tiles_per_seq;
    if (order == kLastFirst) {
      t = tiles_per_seq - 1 - t;
    } else if (order != kNatural) {
      if (order == kMiddleFirst) t = tiles_per_seq - 1 - t;
      t = (t & 1) ? tiles_per_seq - 1 - (t >> 1) : (t >> 1);  // 0, T-1, 1, T-2, ...
    }
    xq = (grp / heads) * tiles_per_seq + t;
    h = grp % heads;
  } else if (fixed) {
    xq = n % nx;
    h = n / nx;
  } else {
    // packed sequences: the work-list holds the tiles longest sequence first; all heads of a tile are
    // dealt before the next tile, so the whole launch runs from long workgroups to short ones
    xq = n / heads;
    h = n % heads;
  }
}

// 16 bytes per lane from global memory straight into LDS: lane l's data lands at lds_base + 16*l
// (lds_base: byte offset in the workgroup's LDS, the same in every lane).  Issued through asm so
// that the compiler keeps no account of it: the kernel waits for these loads itself, with
// wait_vmcnt, and only for the tile it is about to read.  Loads complete in issue order, so the
// compiler's own vmcnt waits, which do not count them, can only wait longer than needed.  M0 is
// a reserved register that cannot be named as a clobber: the block saves it, sets it, uses it and puts
// the old value back, so whatever the compiler itself keeps in M0 survives the block.
__device__ __forceinline__ void dma16(const void* g, uint32_t lds_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
  uint32_t keep;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
               : "=&s"(keep) : "v"(g), "s"(base) : "memory");
}
// One dword per lane, global memory -> LDS at lds_base + 4 * lane.
__device__ __forceinline__ void dma4(const void* g, uint32_t lds_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
  uint32_t keep;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %1, off\n\ts_mov_b32 m0, %0"
               : "=&s"(keep) : "v"(g), "s"(base) : "memory");
}
// The same with the address split into a base that is the same in every lane (it travels in scalar
// registers) and this lane's 32-bit byte offset from it.
__device__ __forceinline__ void dma16s(const void* base, uint32_t lane_off, uint32_t lds_base) {
  const uint32_t lb = __builtin_amdgcn_readfirstlane(lds_base);
  const uint64_t b64 = (uint64_t)(uintptr_t)base;
  const uint32_t blo = __builtin_amdgcn_readfirstlane((uint32_t)b64), bhi = __builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32));
  const uint64_t sb = ((uint64_t)bhi << 32) | blo;
  uint32_t keep;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b32 m0, %0"
               : "=&s"(keep) : "v"(lane_off), "s"(sb), "s"(lb) : "memory");
}
// The same two loads with M0 set and left as it is: for kernels in which nothing else reads M0 (no other direct
// load variant, no LDS-direct or message instructions), where saving and restoring it is two more scalar
// instructions per load.
__device__ __forceinline__ void dma16n(const void* g, uint32_t lds_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(lds_base);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(base) : "memory");
}
__device__ __forceinline__ void dma16sn(const void* base, uint32_t lane_off, uint32_t lds_base) {
  const uint32_t lb = __builtin_amdgcn_readfirstlane(lds_base);
  const uint64_t b64 = (uint64_t)(uintptr_t)base;
  const uint32_t blo = __builtin_amdgcn_readfirstlane((uint32_t)b64), bhi = __builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32));
  const uint64_t sb = ((uint64_t)bhi << 32) | blo;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_off), "s"(sb), "s"(lb) : "memory");
}

// Wait until at most N vector-memory loads of this wave are outstanding (loads complete in issue
// order).  Issued through the builtin rather than asm, so that the compiler's own count of its
// outstanding loads takes the wait into account and it does not wait a second time for a value
// these waits have already covered.  Encoding (gfx9): vmcnt in bits 3:0 and 15:14, expcnt 6:4 and
// lgkmcnt 11:8 left at their maxima (no wait).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
  asm volatile("" ::: "memory");
}

// Padded fixed layout: the rows of `out` outside a batch row's real tokens, written by the workgroup whose tile index t
// covers them in absolute terms (rows [128 t, 128 t + 128), two threads per row of ROW_BYTES): zeros, or `word` = the
// element type's NaN pattern for a batch row the caller marked with a negative token count.
template <int ROW_BYTES>
__device__ __forceinline__ void fill_pad_rows(char* out_bh, int64_t row_stride_bytes, int t, int L, int tok0, int Lb,
                                              uint32_t word, int tid) {
  static_assert(ROW_BYTES % 32 == 0, "two threads per row, 16-byte stores");
  const int row = t * 128 + (tid >> 1);
  if (row >= L || (row >= tok0 && row < tok0 + Lb)) return;
  char* dst = out_bh + (int64_t)row * row_stride_bytes + (tid & 1) * (ROW_BYTES / 2);
  const u32x4 w = {word, word, word, word};
#pragma unroll
  for (int c = 0; c < ROW_BYTES / 32; ++c) *(u32x4*)(dst + 16 * c) = w;
}

// Number of direct loads (dma16 / dma16s) a wave issues per K/V tile of the far-only staging: the waits
// of that staging name this count, so the two are tied together here.
constexpr int kDmaLoadsPerTile = 4;

// Orders this wave's earlier LDS accesses before its later ones (the LDS unit executes one wave's
// operations in order; this only stops the compiler from moving them across).
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// One 64-key tile whose scores leave the MFMA ready for the exponential (the query operand carries the soft-max
// scale and the accumulator started from negm = row_add - (reference point of the row), so sacc = x - reference):
// mask, online soft-max in base 2, O^T += V^T P^T.
// No row maximum on the common path.  The probabilities of the tile are formed
// against the row's current reference point straight away; their sum bounds their maximum, so a
// row whose half-sum stays under 2^kLazyTau needs no new reference point (the same guarantee the
// maximum gives above).  Only when a row fails that test, overflows, or sees its first tile does
// the wave fall back: it recomputes the scores (requery), finds the maximum and moves the
// reference points of those rows onto it.
template <class VT, int D, bool MASK, class VL, class RQ>
__device__ __forceinline__ void softmax_pv_pre2(f32x16 (&sacc)[2], f32x16 (&o_acc)[D / 32], float& m_run, float& l_run,
                                                float row_add, f32x16& negm, const VL& vload, const RQ& requery, int lane,
                                                int j0, int i, int Lb, bool causal) {
  using vfrag = typename VT::frag;
  const int g = lane >> 5;
  auto mask = [&]() __attribute__((always_inline)) {
    if constexpr (MASK) {
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int j = j0 + 32 * jb + 8 * (v >> 2) + 4 * g + (v & 3);
          if (j >= Lb || (causal && j > i)) sacc[jb][v] = -INFINITY;
        }
    }
  };
  vfrag pf[4];
  float l_tile = 0.f;
  auto probs = [&]() __attribute__((always_inline)) {
    l_tile = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      f32x8 pv;
#pragma unroll
      for (int e = 0; e < 8; ++e) pv[e] = __builtin_amdgcn_exp2f(sacc[c >> 1][8 * (c & 1) + e]);
      pf[c] = VT::from_f32(pv);
      l_tile = sum8(pv, l_tile);
    }
  };
  const bool first = m_run == -INFINITY;
  bool slow = __any(first);
  if (!slow) {
    mask();
    probs();
    slow = __any(!(l_tile <= 256.f));  // 2^kLazyTau; also true for an overflow
  }
  if (slow) {
    // both lanes of a row (its two key halves) must move together
    const bool mv = first || wave_half_max(l_tile <= 256.f ? 0.f : 1.f) > 0.f;
    requery(sacc);
    mask();
    float mx = sacc[0][0];
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sacc[jb][v]);
    mx = wave_half_max(mx);
    const float shift = mv ? mx : 0.f;
    const float alpha = mv ? (first ? 0.f : __builtin_amdgcn_exp2f(-shift)) : 1.f;
    if (mv) m_run = (first ? 0.f : m_run) + shift;
    l_run *= alpha;
#pragma unroll
    for (int d = 0; d < D / 32; ++d)
#pragma unroll
      for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
      for (int v = 0; v < 16; ++v) sacc[jb][v] -= shift;
    const float nm = row_add - m_run;
#pragma unroll
    for (int v = 0; v < 16; ++v) negm[v] = nm;
    probs();
  }
  l_run += l_tile;
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int d = 0; d < D / 32; ++d) o_acc[d] = VT::mma(vload(c, d), pf[c], o_acc[d]);
}

}  // namespace fdb
