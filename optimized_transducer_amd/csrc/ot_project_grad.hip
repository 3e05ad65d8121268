// Gradient of the joiner's output projection with respect to its weight and bias (gfx950 MFMA).
//
// logits = x W^T + b on the packed rows (README.md:176-177 of the reference; forward in
// ot_project.hip), so with g = d loss / d logits (rows, V), the loss's own output:
//     grad_W = g^T x   (V, D)        grad_b = sum over the rows of g   (V)
// Both operands are stored with the contraction index - the packed row, hundreds of
// thousands of them - as their SLOW index, which is the one arrangement a matrix
// instruction cannot take its operands from directly: a lane wants 8 consecutive k for one
// m.  The tiles therefore go to LDS as they lie in memory ([row][column], 16-byte pieces)
// and are read back with ds_read_b64_tr_b16, which hands every lane of a group of 16 the
// four values of ITS column out of a 4 x 16 block: two such reads are one operand of
// v_mfma_f32_32x32x16.
//
// Shape of the computation.  A workgroup of 4 waves owns a 256 x 256 tile of grad_W and a
// slice of the packed rows; the waves form a 2 x 2 grid, a wave holds 128 x 128 of the tile
// in 16 accumulator tiles (256 accumulator registers: one workgroup per compute unit).  g
// and x stream through LDS in stages of 32 rows (two buffers, one barrier per stage); the
// global loads of a stage are issued four stages ahead into a ring of registers.  The
// workgroup that owns the first 256 columns of D also adds up its g tile by columns for
// grad_b, in the registers the tile passes through on its way to LDS.  The four tiles of a
// slice run on the same XCD at the same time, so that its L2 serves the second reader of
// every piece of g and x.  Every slice leaves a partial result; a second kernel adds the
// slices in a fixed order.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ot_device.hip.h"
#include "ot_transducer.h"

namespace ot {

typedef __bf16 wg_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 wg_f16x8 __attribute__((ext_vector_type(8)));
typedef float wg_f32x16 __attribute__((ext_vector_type(16)));
typedef short wg_i16x4 __attribute__((ext_vector_type(4)));
typedef short wg_i16x8 __attribute__((ext_vector_type(8)));

constexpr int kWgTile = 256;            // edge of a workgroup's tile of grad_W
constexpr int kWgRows = 32;             // packed rows per stage
constexpr int kWgPitch = kWgTile + 32;  // LDS row pitch in elements: 144 dwords, so that the 4 rows of a
                                        // transposing read fall into 4 different quarters of the 64 banks
constexpr int kWgThreads = 256;
constexpr int kWgPieces = kWgRows * kWgTile / 8 / kWgThreads;  // 16-byte pieces per thread and operand: 4
constexpr int kWgAhead = 4;             // stages of global loads in flight

template <class E>
__device__ __forceinline__ wg_f32x16 wg_mfma(wg_i16x8 a, wg_i16x8 b, wg_f32x16 c);
template <>
__device__ __forceinline__ wg_f32x16 wg_mfma<BF16>(wg_i16x8 a, wg_i16x8 b, wg_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(wg_bf16x8, a),
                                                 __builtin_bit_cast(wg_bf16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ wg_f32x16 wg_mfma<F16>(wg_i16x8 a, wg_i16x8 b, wg_f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(wg_f16x8, a),
                                                __builtin_bit_cast(wg_f16x8, b), c, 0, 0, 0);
}

// Half an operand of one 32-wide tile: `q` points at this lane's place in the first of 4
// rows.  One read transposes a block of 4 rows x 16 columns per group of 16 lanes: lane p of
// the group fetches row p / 4, columns 4 (p % 4) .. + 3 and receives column p of all 4 rows.
// With lane l = 32 kg + 16 h + p reading rows 8 kg + .. of the columns 16 h + .., two reads
// 4 rows apart are the 8 consecutive k of column l % 32 that v_mfma_f32_32x32x16 wants.
__device__ __forceinline__ wg_i16x4 wg_read_tr(const unsigned short *q) {
  typedef wg_i16x4 __attribute__((address_space(3))) * lds_ptr;
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)q);
}
__device__ __forceinline__ wg_i16x8 wg_join(const wg_i16x4 (&v)[2]) {
  return wg_i16x8{v[0][0], v[0][1], v[0][2], v[0][3], v[1][0], v[1][1], v[1][2], v[1][3]};
}

// Workgroup id -> (slice, tile): the tiles of a slice share an XCD (workgroup i runs on XCD
// i % 8) and are dispatched within 8 * tiles consecutive ids.  slices is a multiple of 8.
template <class E>
__global__ __launch_bounds__(kWgThreads) void joiner_weight_grad_kernel(
    const unsigned short *__restrict__ g, const unsigned short *__restrict__ x, int64_t rows,
    int V, int D, int64_t rows_per_slice, int m_tiles, int n_tiles, float *__restrict__ partial_w,
    float *__restrict__ partial_b) {
  __shared__ __attribute__((aligned(16))) unsigned short s_g[2][kWgRows][kWgPitch];
  __shared__ __attribute__((aligned(16))) unsigned short s_x[2][kWgRows][kWgPitch];
  __shared__ float s_b[kWgThreads / 32][kWgTile];
  const int tid = threadIdx.x, lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles = m_tiles * n_tiles;
  const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
  const int tile = q % tiles;
  const int slice = (q / tiles) * 8 + xcd;
  const int mt = tile / n_tiles, nt = tile - mt * n_tiles;
  const int m0 = mt * kWgTile, n0 = nt * kWgTile;
  const int64_t r0 = (int64_t)slice * rows_per_slice;
  const int64_t r1 = min(rows, r0 + rows_per_slice);
  const int nrows = (int)max((int64_t)0, r1 - r0);
  const int nstages = (nrows + kWgRows - 1) / kWgRows;

  // the slice's rows as raw buffers: rows behind its end read as zeros
  const __amdgpu_buffer_rsrc_t g_buf = make_buffer(g + r0 * V, (unsigned)nrows * (unsigned)V * 2u);
  const __amdgpu_buffer_rsrc_t x_buf = make_buffer(x + r0 * D, (unsigned)nrows * (unsigned)D * 2u);
  // this thread's pieces of a stage: rows tid / 32 + 8 i, columns 8 (tid % 32) .. + 7
  const int prow = tid >> 5, pcol = (tid & 31) * 8;
  const bool g_ok = m0 + pcol < V, x_ok = n0 + pcol < D;  // V and D are multiples of 8
  unsigned g_off = g_ok ? (unsigned)(prow * V + m0 + pcol) * 2u : 0xFFFFFFFFu;
  unsigned x_off = x_ok ? (unsigned)(prow * D + n0 + pcol) * 2u : 0xFFFFFFFFu;
  const unsigned g_step = g_ok ? (unsigned)(8 * V) * 2u : 0u, x_step = x_ok ? (unsigned)(8 * D) * 2u : 0u;
  const unsigned g_stage = g_ok ? (unsigned)(kWgRows * V) * 2u : 0u;
  const unsigned x_stage = x_ok ? (unsigned)(kWgRows * D) * 2u : 0u;

  u32x4 gq[kWgAhead][kWgPieces], xq[kWgAhead][kWgPieces];
  // load t of a stage: piece t / 2 of g (t even) or x (t odd)
  auto issue = [&](u32x4(&gr)[kWgPieces], u32x4(&xr)[kWgPieces], int t) {
    const int i = t >> 1;
    if (t & 1)
      xr[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(x_buf, x_off + i * x_step, 0, 0));
    else
      gr[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(g_buf, g_off + i * g_step, 0, 0));
    if (t == 2 * kWgPieces - 1) {
      g_off += g_stage;
      x_off += x_stage;
    }
  };
  // piece t / 2 of g (t even) or x (t odd) into LDS
  auto deposit = [&](const u32x4(&gr)[kWgPieces], const u32x4(&xr)[kWgPieces], int buf, int t) {
    const int i = t >> 1;
    if (t & 1)
      *reinterpret_cast<u32x4 *>(&s_x[buf][prow + 8 * i][pcol]) = xr[i];
    else
      *reinterpret_cast<u32x4 *>(&s_g[buf][prow + 8 * i][pcol]) = gr[i];
  };
  // column sums of g for grad_b from the same registers, rows ascending: part t adds the
  // two columns of dword t % 4 of piece t / 4.  Only the workgroup of the first tile of D
  // keeps the sums; all of them add, which keeps the loop free of branches (sharing the
  // pieces among the workgroups that load the same tile of g, with a branch around each
  // part, was measured and is slower).
  float bsum[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) bsum[e] = 0.f;
  auto add_up = [&](const u32x4(&gr)[kWgPieces], int t) {
    const int e = t & 3;
    const unsigned w = gr[t >> 2][e];
    bsum[2 * e] += to_float<E>((unsigned short)(w & 0xFFFFu));
    bsum[2 * e + 1] += to_float<E>((unsigned short)(w >> 16));
  };

  // operands of a k-step (16 rows): a[i] for the 4 tiles of g, b[j] for the 4 tiles of x,
  // as 16 reads in the order a0 b0 b1 b2 b3 a1 a2 a3 (the order the products need them in)
  const int fp = lane & 15, fh = (lane >> 4) & 1, fkg = lane >> 5;
  const int frag = (8 * fkg + (fp >> 2)) * kWgPitch + 16 * fh + 4 * (fp & 3);
  const int a_frag = frag + 128 * wm, b_frag = frag + 128 * wn;
  auto fetch = [&](wg_i16x4(&a)[4][2], wg_i16x4(&b)[4][2], int buf, int ks, int r) {
    const int o = r >> 1, half = r & 1, row = 16 * ks + 4 * half;
    if (o == 0)
      a[0][half] = wg_read_tr(&s_g[buf][row][0] + a_frag);
    else if (o <= 4)
      b[o - 1][half] = wg_read_tr(&s_x[buf][row][0] + b_frag + 32 * (o - 1));
    else
      a[o - 4][half] = wg_read_tr(&s_g[buf][row][0] + a_frag + 32 * (o - 4));
  };

  wg_f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // stages 0 .. kWgAhead-1 on their way, stage 0 in LDS, its first k-step in registers
  wg_i16x4 fa[4][2], fb[4][2], na[4][2], nb[4][2];
#pragma unroll
  for (int a = 0; a < kWgAhead; ++a)
#pragma unroll
    for (int t = 0; t < 2 * kWgPieces; ++t) issue(gq[a], xq[a], t);
#pragma unroll
  for (int t = 0; t < 2 * kWgPieces; ++t) deposit(gq[0], xq[0], 0, t);
#pragma unroll
  for (int t = 0; t < 4 * kWgPieces; ++t) add_up(gq[0], t);
  lds_barrier();
#pragma unroll
  for (int r = 0; r < 16; ++r) fetch(fa, fb, 0, 0, r);

  // One wave per SIMD: whatever the wave waits for, the matrix core waits for too.  So
  // everything else is dealt out over the 32 products of a stage by hand, and the fences
  // keep the compiler from gathering it again.  The four waves run in step (one barrier per
  // stage) and share the compute unit's address path (a global load: 16 clocks) and LDS
  // write port (16 bytes per lane: 13 clocks), so loads and LDS writes are spread over the
  // whole stage rather than bunched behind consecutive products:
  //   global load t of stage s + kWgAhead     after product 4 t             (t = 0 .. 7)
  //   piece t of stage s + 1 into LDS         after product 3 t             (t = 0 .. 7)
  //   operand reads of k-step 1               after products 0 .. 15, one each
  //   column sums of stage s + 1              after products 16 .. 31
  //   the barrier                             after product 23
  //   operand reads of stage s + 1, k-step 0  after products 24 .. 31, two each
  // The copies go to the other LDS buffer, whose readers passed the previous barrier.  The
  // stages are rounded up to a multiple of kWgAhead: a stage behind the slice's end loads
  // zeros and adds zeros.
  for (int s = 0; s < nstages; s += kWgAhead) {
#pragma unroll
    for (int a = 0; a < kWgAhead; ++a) {
      const int cur = (s + a) & 1, nxt = cur ^ 1;
#pragma unroll
      for (int slot = 0; slot < 32; ++slot) {
        const int t = slot & 15;
        if (slot < 16)
          acc[t >> 2][t & 3] = wg_mfma<E>(wg_join(fa[t >> 2]), wg_join(fb[t & 3]), acc[t >> 2][t & 3]);
        else
          acc[t >> 2][t & 3] = wg_mfma<E>(wg_join(na[t >> 2]), wg_join(nb[t & 3]), acc[t >> 2][t & 3]);
        if (slot % 4 == 0) issue(gq[a], xq[a], slot / 4);
        if (slot % 3 == 0 && slot / 3 < 2 * kWgPieces)
          deposit(gq[(a + 1) % kWgAhead], xq[(a + 1) % kWgAhead], nxt, slot / 3);
        if (slot < 16) {
          fetch(na, nb, cur, 1, t);
        } else {
          add_up(gq[(a + 1) % kWgAhead], t);
          if (slot == 23) lds_barrier();
          if (slot >= 24) {
            fetch(fa, fb, nxt, 0, 2 * (slot - 24));
            fetch(fa, fb, nxt, 0, 2 * (slot - 24) + 1);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // partial tile: accumulator r of a lane is row 8 (r / 4) + 4 (lane / 32) + r % 4 and column
  // lane % 32 of its 32 x 32 tile
  float *const out = partial_w + ((int64_t)slice * (m_tiles * kWgTile) + m0) * (int64_t)(n_tiles * kWgTile) + n0;
  const int64_t out_pitch = (int64_t)n_tiles * kWgTile;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = 128 * wm + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        const int n = 128 * wn + 32 * j + (lane & 31);
        out[m * out_pitch + n] = acc[i][j][r];
      }
  if (nt == 0) {
    // the 8 threads of a column block, rows ascending
#pragma unroll
    for (int e = 0; e < 8; ++e) s_b[prow][pcol + e] = bsum[e];
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < kWgThreads / 32; ++k) t += s_b[k][tid];
    partial_b[(int64_t)slice * (m_tiles * kWgTile) + m0 + tid] = t;
  }
}

// grad_W[m][n] = sum over the slices, in slice order, rounded once to the weight's type;
// grad_b[m] likewise in float32.
template <class E>
__global__ __launch_bounds__(kBlock) void joiner_weight_grad_reduce_kernel(
    const float *__restrict__ partial_w, const float *__restrict__ partial_b, int slices, int V,
    int D, int m_pad, int n_pad, unsigned short *__restrict__ grad_w, float *__restrict__ grad_b) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < (int64_t)V * D) {
    const int m = (int)(i / D), n = (int)(i - (int64_t)m * D);
    float t = 0.f;
    for (int s = 0; s < slices; ++s) t += partial_w[((int64_t)s * m_pad + m) * n_pad + n];
    grad_w[i] = from_float<E>(t);
  }
  if (grad_b && i < V) {
    float t = 0.f;
    for (int s = 0; s < slices; ++s) t += partial_b[(int64_t)s * m_pad + i];
    grad_b[i] = t;
  }
}

static inline int wg_launch_status() { return (int)hipGetLastError(); }

struct WgPlan {
  int m_tiles, n_tiles, slices;
  int64_t rows_per_slice;
};
static WgPlan wg_plan(int64_t rows, int V, int D) {
  WgPlan p;
  p.m_tiles = (V + kWgTile - 1) / kWgTile;
  p.n_tiles = (D + kWgTile - 1) / kWgTile;
  int cus = 256, device = 0;
  if (hipGetDevice(&device) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
    cus = 256;
  // one workgroup per compute unit, slices a multiple of 8, at least one stage per slice
  int64_t slices = cus / (p.m_tiles * p.n_tiles);
  slices = slices / 8 * 8;
  if (slices < 8) slices = 8;
  int64_t per = (rows + slices - 1) / slices;
  per = (per + kWgRows - 1) / kWgRows * kWgRows;
  p.slices = (int)slices;
  p.rows_per_slice = per;
  return p;
}

}  // namespace ot

using namespace ot;

extern "C" {

size_t ot_joiner_weight_grad_workspace_bytes(int64_t rows, int32_t V, int32_t D) {
  if (rows <= 0 || V <= 0 || D <= 0) return 0;
  const WgPlan p = wg_plan(rows, V, D);
  const size_t m_pad = (size_t)p.m_tiles * kWgTile, n_pad = (size_t)p.n_tiles * kWgTile;
  return (size_t)p.slices * (m_pad * n_pad + m_pad) * sizeof(float);
}

int ot_joiner_weight_grad(const void *grad_logits, const void *x, int32_t dtype, int64_t rows,
                          int32_t V, int32_t D, void *workspace, size_t workspace_bytes,
                          void *grad_weight, float *grad_bias, void *stream) {
  if (!grad_logits || !x || !workspace || !grad_weight || rows <= 0 || rows > INT32_MAX || V <= 0 ||
      D <= 0 || (dtype != OT_DTYPE_F16 && dtype != OT_DTYPE_BF16))
    return OT_E_BAD_ARG;
  if (V % 8 != 0 || D % 8 != 0) return OT_E_BAD_ARG;
  if ((reinterpret_cast<uintptr_t>(grad_logits) & 15) || (reinterpret_cast<uintptr_t>(x) & 15) ||
      (reinterpret_cast<uintptr_t>(workspace) & 15) || (reinterpret_cast<uintptr_t>(grad_weight) & 1) ||
      (reinterpret_cast<uintptr_t>(grad_bias) & 3))
    return OT_E_MISALIGNED;
  if (workspace_bytes < ot_joiner_weight_grad_workspace_bytes(rows, V, D)) return OT_E_BAD_ARG;
  const WgPlan p = wg_plan(rows, V, D);
  // a slice's rows are addressed with 32-bit byte offsets
  if (p.rows_per_slice * (int64_t)(V > D ? V : D) * 2 + ((int64_t)kWgAhead + 2) * kWgRows * (V > D ? V : D) * 2 >
      (int64_t)0x7FFFFFFF)
    return OT_E_TOO_LONG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int m_pad = p.m_tiles * kWgTile, n_pad = p.n_tiles * kWgTile;
  float *partial_w = static_cast<float *>(workspace);
  float *partial_b = partial_w + (size_t)p.slices * m_pad * n_pad;
  const unsigned blocks = (unsigned)(p.slices * p.m_tiles * p.n_tiles);
  const unsigned short *gp = static_cast<const unsigned short *>(grad_logits);
  const unsigned short *xp = static_cast<const unsigned short *>(x);
  unsigned short *wp = static_cast<unsigned short *>(grad_weight);
  const int64_t cells = (int64_t)V * D;
  const unsigned rblocks = (unsigned)((cells + kBlock - 1) / kBlock);
  if (dtype == OT_DTYPE_BF16) {
    hipLaunchKernelGGL(joiner_weight_grad_kernel<BF16>, dim3(blocks), dim3(kWgThreads), 0, s, gp, xp,
                       rows, V, D, p.rows_per_slice, p.m_tiles, p.n_tiles, partial_w, partial_b);
    hipLaunchKernelGGL(joiner_weight_grad_reduce_kernel<BF16>, dim3(rblocks), dim3(kBlock), 0, s,
                       partial_w, partial_b, p.slices, V, D, m_pad, n_pad, wp, grad_bias);
  } else {
    hipLaunchKernelGGL(joiner_weight_grad_kernel<F16>, dim3(blocks), dim3(kWgThreads), 0, s, gp, xp,
                       rows, V, D, p.rows_per_slice, p.m_tiles, p.n_tiles, partial_w, partial_b);
    hipLaunchKernelGGL(joiner_weight_grad_reduce_kernel<F16>, dim3(rblocks), dim3(kBlock), 0, s,
                       partial_w, partial_b, p.slices, V, D, m_pad, n_pad, wp, grad_bias);
  }
  return wg_launch_status();
}

}  // extern "C"
