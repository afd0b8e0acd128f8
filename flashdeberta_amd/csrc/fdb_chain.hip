// The chain of the backward through the position tables, both products in one pass over the score gradients.
//
// The backward kernels leave the score gradients G = d c2p (or d p2c) as a tensor [matrix][row][2S], one matrix per
// head and term, one row per token.  The chain rule through score = x . pos[delta] (x: the token's q or k row, pos:
// the table K_r or Q_r of the head) needs two products of G:
//     dx   [row][d]   += sum_delta G[row][delta] * pos[delta][d]      (back into dq / dk, on top of the content part)
//     dpos [delta][d]  = sum_row   G[row][delta] * x[row][d]          (the table's gradient, a reduction over the tokens)
// which the reference leaves to autograd as two matrix products per term (the backward of model.py:189-192, where
// the score tensors are made) -- two reads of the largest tensor of the backward.  Here a workgroup walks a share of
// a matrix's rows 32 at a time: the 32 x 2S tile of G goes from global memory straight into one of two LDS buffers
// (the next tile on its way while this one is used) and feeds both products from there.  The workgroup is two teams
// of four waves, one per product, so that every SIMD holds a wave of each:
//   * dpos (waves 0-3): M = delta, N = d, K = row -- both operands are read transposed from row-major LDS tiles
//     (ds_read_b64_tr_b16), wave w owning table-row blocks 4w .. 4w+3; the tile of x (rows of any stride: q and k are
//     read where they lie) passes through registers into padded LDS rows.  Every workgroup keeps its share of dpos in
//     registers (fp32, 32 KB of accumulators per wave) and writes it once, as one of `parts` partial sums the caller
//     adds up.
//   * dx (waves 4-7): computed transposed, M = d, N = row, K = delta, so that a lane ends up with four neighbouring d
//     of one row (8-byte stores).  A wave takes one 32-wide block of d and half of the table rows and keeps its share
//     of pos, transposed, in 64 registers for the life of the workgroup; the operand from G is a plain 16-byte row
//     read.  The upper two waves hand their halves to the lower two through LDS one tile late (the barrier that opens
//     the next tile orders the hand-over), and those add both halves onto the rows of dx in memory, asked for when
//     the step begins and used when it ends: fp32 accumulation over the kernels' content part and one rounding, as
//     a GEMM with beta = 1 would.
// Both teams run the same number of barriers (one per tile, one after the last).  The launch moves G once, x once and
// dx twice: 1.1 GB at the bench shape in 0.26 ms, which is what the memory system gives this pattern; the two GEMMs it
// replaces take 0.44 ms.
//
// Shapes: head_dim 64, 2S = 512, rows a multiple of 32, bf16 or fp16; the entry point refuses anything else and the
// Python operator then takes the two GEMMs.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "fdb_device.h"
#include "fdb_kernels.h"
#include "../../include/fdb.h"

using namespace fdb;

namespace {

constexpr int kChainThreads = 512;           // two teams of four waves: one per product
constexpr int kChainRows = 32;               // rows of G per tile
constexpr int kChainS2 = 512, kChainD = 64;
constexpr int kRowX = kChainD * 2 + 16;      // LDS row strides: 16 bytes of padding keep the reads of a column of rows off one bank
constexpr int kRowG = kChainS2 * 2 + 16;
constexpr int kBytesG = kChainRows * kRowG;  // 33280 per buffer
constexpr int kBytesX = kChainRows * kRowX;  //  4608 per buffer
constexpr int kBytesR = 2 * 16 * 64 * 4;     //  8192 per buffer: the upper waves' halves of dx^T, [wave][register][lane]
constexpr int kChainLds = 2 * kBytesG + 2 * kBytesX + 2 * kBytesR;
static_assert(kChainLds <= 160 * 1024, "LDS budget");

template <class QT>
__global__ __launch_bounds__(kChainThreads, 1) void fdb_chain_kernel(const FdbChainParams p) {
  using frag = typename QT::frag;
  using ST = typename QT::scratch_t;
  typedef ST st4 __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* G_s = smem;                       // two buffers of [32][kRowG]
  char* X_s = G_s + 2 * kBytesG;          // two buffers of [32][kRowX]
  float* R_s = (float*)(X_s + 2 * kBytesX);  // two buffers of [2][16][64]
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, li = lane & 31, g = lane >> 5;
  const int m = blockIdx.y, part = blockIdx.x;
  const int64_t tiles = p.rows / kChainRows;
  const int64_t t0 = (int64_t)part * p.tiles_per_part;
  const int64_t t1 = t0 + p.tiles_per_part < tiles ? t0 + p.tiles_per_part : tiles;
  const char* gm = p.g + (int64_t)m * p.rows * (kChainS2 * 2);
  const uint32_t lds0 = (uint32_t)(uintptr_t)(LDS_AS char*)smem;
  // a row of G is 1 KB: one direct load of a wave (16 bytes per lane); wave w of eight stages rows 4w .. 4w+3 of a tile
  auto g_dma = [&](int64_t t, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = 4 * wave + r;
      dma16(gm + (t * kChainRows + row) * (kChainS2 * 2) + lane * 16, lds0 + buf * kBytesG + row * kRowG);
    }
  };
  // Both teams run the same number of barriers: one per tile and one after the last.
  if (wave < 4) {
    // ---- dpos = G^T x: wave w owns table-row blocks 4w .. 4w+3, all of d ------------------------------------------
    const char* xm = (m < p.split ? p.x + (int64_t)m * p.x_sm * 2 : p.x2 + (int64_t)(m - p.split) * p.x_sm * 2);
    const int64_t x_row = p.x_sr * 2;   // bytes between the rows of x
    f32x16 acc_pos[4][2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc_pos[j][nb][v] = 0.f;
    // the tile of x: 32 rows of eight chunks, one chunk per thread of this team, through a register into the padded rows
    u32x4 xreg = {0u, 0u, 0u, 0u};
    auto x_load = [&](int64_t t) __attribute__((always_inline)) {
      xreg = *(const u32x4*)(xm + (t * kChainRows + (tid >> 3)) * x_row + (tid & 7) * 16);
    };
    if (t0 < t1) {
      g_dma(t0, 0);
      x_load(t0);
    }
    int buf = 0;
    for (int64_t t = t0; t < t1; ++t, buf ^= 1) {
      *(u32x4*)(X_s + buf * kBytesX + (tid >> 3) * kRowX + (tid & 7) * 16) = xreg;
      wait_vmcnt<0>();   // this wave's rows of the tile have landed
      __syncthreads();   // ... and everybody's; every wave is done with the other buffers
      if (t + 1 < t1) {
        g_dma(t + 1, buf ^ 1);
        x_load(t + 1);
      }
      const char* Gt = G_s + buf * kBytesG;
      const char* Xt = X_s + buf * kBytesX;
#pragma unroll
      for (int c = 0; c < 2; ++c) {   // two contraction steps of 16 rows
        const frag bx0 = VtLoad<QT>::get(Xt, kRowX, c, 0, lane), bx1 = VtLoad<QT>::get(Xt, kRowX, c, 1, lane);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const frag a = VtLoad<QT>::get(Gt, kRowG, c, 4 * wave + j, lane);
          acc_pos[j][0] = QT::mma(a, bx0, acc_pos[j][0]);
          acc_pos[j][1] = QT::mma(a, bx1, acc_pos[j][1]);
        }
      }
    }
    if (t0 < t1) __syncthreads();
    // this workgroup's partial sum of dpos: [part][matrix][delta][d], fp32
    float* out = p.parts_out + ((int64_t)part * p.matrices + m) * (kChainS2 * kChainD);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int delta = 32 * (4 * wave + j) + 8 * (v >> 2) + 4 * g + (v & 3);
          out[delta * kChainD + 32 * nb + li] = acc_pos[j][nb][v];
        }
  } else {
    // ---- dx^T += pos^T G^T: wave u = wave - 4 takes block u % 2 of d and half u / 2 of the table rows ---------------
    const int u = wave - 4;
    char* dxm = (m < p.split ? p.dx + (int64_t)m * p.dx_sm * 2 : p.dx2 + (int64_t)(m - p.split) * p.dx_sm * 2);
    const int64_t dx_row = p.dx_sr * 2;   // bytes between the rows of dx
    const char* pm = p.pos + (int64_t)m * (kChainS2 * kChainD * 2);
    // This wave's share of the table, transposed, as the sixteen A operands of its product: column 32 (u % 2) + li,
    // table rows 256 (u / 2) + 16 c + 8 g + 0..7.  64 registers for the life of the workgroup, gathered once.
    frag pa[16];
    {
      const char* col = pm + ((256 * (u >> 1) + 8 * g) * kChainD + 32 * (u & 1) + li) * 2;
#pragma unroll
      for (int c = 0; c < 16; ++c) {
        s16x8 w;
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = *(const short*)(col + (16 * c + e) * (kChainD * 2));
        pa[c] = __builtin_bit_cast(frag, w);
      }
    }
    // Waves 4 and 5 complete the rows of dx of a tile one tile late: their own half of the table rows (kept in
    // registers) plus the half that wave + 2 left in LDS, added onto the rows in memory and rounded once.
    // The rows are asked for when the next tile's step begins and used when it ends, behind its products.
    f32x16 dx_keep = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    st4 dx_old[4];
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) dx_old[q4] = st4{(ST)0.f, (ST)0.f, (ST)0.f, (ST)0.f};
    bool have_prev = false;
    auto dx_ptr = [&](int64_t t, int q4) __attribute__((always_inline)) -> char* {
      return dxm + (t * kChainRows + li) * dx_row + (32 * u + 8 * q4 + 4 * g) * 2;
    };
    auto request_dx = [&](int64_t t) __attribute__((always_inline)) {
      if (u >= 2) return;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) dx_old[q4] = *(const st4*)dx_ptr(t, q4);
    };
    auto finish_dx = [&](int64_t t, int rbuf) __attribute__((always_inline)) {
      if (u >= 2) return;
      const float* r = R_s + rbuf * (kBytesR / 4) + u * (16 * 64) + lane;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const st4 old = dx_old[q4];
        QT::store4(dx_ptr(t, q4), dx_keep[4 * q4] + r[64 * (4 * q4)] + (float)old[0], dx_keep[4 * q4 + 1] + r[64 * (4 * q4 + 1)] + (float)old[1],
                   dx_keep[4 * q4 + 2] + r[64 * (4 * q4 + 2)] + (float)old[2], dx_keep[4 * q4 + 3] + r[64 * (4 * q4 + 3)] + (float)old[3]);
      }
    };
    if (t0 < t1) g_dma(t0, 0);
    int buf = 0;
    for (int64_t t = t0; t < t1; ++t, buf ^= 1) {
      wait_vmcnt<0>();   // this wave's rows of the tile have landed
      __syncthreads();   // ... and everybody's; every wave is done with the other buffers
      if (have_prev) request_dx(t - 1);
      if (t + 1 < t1) g_dma(t + 1, buf ^ 1);
      const char* Gt = G_s + buf * kBytesG;
      f32x16 acc0 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, acc1 = acc0;
      const char* pb = Gt + li * kRowG + (256 * (u >> 1) + 8 * g) * 2;
#pragma unroll
      for (int c = 0; c < 16; c += 2) {   // sixteen contraction steps in two chains
        acc0 = QT::mma(pa[c], QT::load(pb + 32 * c), acc0);
        acc1 = QT::mma(pa[c + 1], QT::load(pb + 32 * c + 32), acc1);
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) acc0[v] += acc1[v];
      if (have_prev) finish_dx(t - 1, buf ^ 1);
      if (u >= 2) {
        float* r = R_s + buf * (kBytesR / 4) + (u - 2) * (16 * 64) + lane;
#pragma unroll
        for (int v = 0; v < 16; ++v) r[64 * v] = acc0[v];
      } else {
        dx_keep = acc0;
      }
      have_prev = true;
    }
    if (have_prev) {
      __syncthreads();   // the upper waves' halves of the last tile are in LDS
      request_dx(t1 - 1);
      finish_dx(t1 - 1, buf ^ 1);
    }
  }
}

template <class QT>
int launch_chain(const FdbChainParams& p, hipStream_t stream) {
  auto kern = fdb_chain_kernel<QT>;
  static std::atomic<uint64_t> lds_set{0};
  hipError_t e = fdb_set_lds_once((const void*)kern, kChainLds, lds_set);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(kern, dim3((unsigned)p.parts, (unsigned)p.matrices), dim3(kChainThreads), kChainLds, stream, p);
  return (int)hipGetLastError();
}

}  // namespace

int fdb_launch_chain(const FdbChainParams& p, int dtype, void* stream) {
  switch (dtype) {
    case FDB_BF16: return launch_chain<Bf16Tr>(p, (hipStream_t)stream);
    case FDB_F16: return launch_chain<F16Tr>(p, (hipStream_t)stream);
    default: return FDB_ERR_DTYPE;
  }
}
