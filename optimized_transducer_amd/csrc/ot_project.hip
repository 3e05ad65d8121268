// Output projection of the joiner fused with the loss's denominators (gfx950 MFMA).
//
// The caller of the reference computes logits = Linear(tanh(enc + dec)) on the
// packed rows (README.md:166-177) and hands them to the loss, whose first step
// reads all of them again for logits.logsumexp(1) (cuda.cu:427).  Here the
// projection of 2-byte activations x (rows, D) with the weight W (V, D) and the
// bias runs on the matrix cores with float32 accumulation, and the per-row
// log-sum-exp of exactly the values that are stored comes out of the accumulators:
// the loss then starts from its gather step and the logits are read once, by the
// gradient pass, instead of twice.
//
// Shape of the computation.  A workgroup of 4 waves owns 128 packed rows and walks
// over the vocabulary in passes of 256 columns; the waves form a 2 x 2 grid, a wave
// holds a 128 x 64 block of logits^T in 8 accumulator tiles of 32 x 32
// (v_mfma_f32_32x32x16).  The product is formed transposed (vocabulary along the
// tile's rows, packed rows along its columns) because an accumulator lane then
// holds 16 values of ONE packed row per tile: the running (max, sum) of the row
// stays in that lane, with no cross-lane reduction until the very end, where the
// lane's partner 32 lanes up and the 2 waves of the row are merged.  W and x
// stream through LDS in stages of 32 k-values (two buffers, 16-byte slots
// XOR-swizzled against bank conflicts); the global loads of a stage are issued two
// stages ahead into one of two register sets, because one stage of matrix work is
// shorter than a trip to memory.  The bias initialises the accumulators.  The
// stores go through a small wave-private LDS tile that turns the accumulator layout
// into whole 128-byte pieces of rows.  Workgroups are persistent (two per compute
// unit), so the loads of the next 128 rows are in flight while the last pass of the
// current ones is stored.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ot_device.hip.h"
#include "ot_transducer.h"

namespace ot {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

// bit patterns by value (a bit cast applied directly to a vector element reads element 0)
__device__ __forceinline__ unsigned as_u32(float v) { return __builtin_bit_cast(unsigned, v); }
__device__ __forceinline__ float as_f32(unsigned v) { return __builtin_bit_cast(float, v); }

constexpr int kProjRows = 128;     // packed rows per workgroup (2 waves of 64)
constexpr int kProjCols = 256;     // vocabulary columns per pass (2 waves of 128)
constexpr int kProjK = 32;         // k-values per LDS stage
constexpr int kProjThreads = 256;
// ordinary (cached) stores: rows whose pitch is not a multiple of 128 bytes are written in
// partial lines, for which the non-temporal policies are 20-90 % slower here
constexpr int kProjStoreAux = 0;
constexpr int kProjWBytes = kProjCols * kProjK * 2;
constexpr int kProjXBytes = kProjRows * kProjK * 2;
constexpr int kProjStageBytes = kProjWBytes + kProjXBytes;
constexpr int kProjWPieces = kProjWBytes / 16 / kProjThreads;  // 16-byte pieces per thread: 4
constexpr int kProjXPieces = kProjXBytes / 16 / kProjThreads;  // 2
// store tile of a wave: 32 rows x 32 float columns, rows 9 sixteen-byte units apart
constexpr int kProjTilePitch = 32 * 4 + 16;
constexpr int kProjTileBytes = 32 * kProjTilePitch;

template <class E>
__device__ __forceinline__ f32x16 mfma_32x32x16(u32x4 a, u32x4 b, f32x16 c);
template <>
__device__ __forceinline__ f32x16 mfma_32x32x16<BF16>(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16 mfma_32x32x16<F16>(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// one stage's worth of global data of a thread, on its way to LDS
struct ProjStage {
  u32x4 w[kProjWPieces];
  u32x4 x[kProjXPieces];
};

// E: element type of x and W.  OUT_F32: logits are float32, else of type E.
// SV: elements per store (SV * element size divides the row pitch and the base).
// D is a multiple of 64 (an even number of stages).
template <class E, bool OUT_F32, int SV>
__global__ __launch_bounds__(kProjThreads, 2) void joiner_project_kernel(
    const unsigned short *__restrict__ x, const unsigned short *__restrict__ w,
    const float *__restrict__ bias, int64_t rows, int D, int V, void *__restrict__ logits,
    float *__restrict__ den, int paired) {
  __shared__ __attribute__((aligned(16))) unsigned char s_stage[2 * kProjStageBytes];
  __shared__ float2 s_part[2][kProjRows];
  __shared__ __attribute__((aligned(16))) float s_bias[kProjCols];  // the pass's starting values
  __shared__ __attribute__((aligned(16))) unsigned char s_tile[4 * kProjTileBytes];
  constexpr unsigned kOutBytes = OUT_F32 ? 4u : 2u;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int c = lane & 31, h = lane >> 5;
  // Persistent workgroups: workgroup g takes the 128-row tiles g, g + gridDim.x, ... and
  // all passes of each; the loads of the next tile's first stages are already in flight
  // while the current tile's last pass is stored.
  // Paired (the caller lends room for one partial log-sum-exp per row and pass): a workgroup
  // takes ONE pass of its tiles, and the workgroups that take the other passes of the same
  // tiles run beside it on the same XCD (ids 8 apart), so that x leaves HBM once and the
  // other readers are served by that XCD's L2; `den` then holds the parts, pass-major.
  const int64_t ntiles = (rows + kProjRows - 1) / kProjRows;
  const int npasses_all = (V + kProjCols - 1) / kProjCols;
  int64_t tile_first = blockIdx.x, tile_stride = gridDim.x;
  int pass_first = 0, pass_count = npasses_all;
  if (paired) {
    const int k = (int)blockIdx.x >> 3;
    pass_first = k % npasses_all;
    pass_count = 1;
    tile_first = (int64_t)(k / npasses_all) * 8 + (blockIdx.x & 7);
    tile_stride = (int64_t)(gridDim.x / 8 / npasses_all) * 8;
    den += (int64_t)pass_first * rows;
  }
  const int pass_end = pass_first + pass_count;
  // the weight and the bias as raw buffers: vocabulary entries past V read as zeros
  const __amdgpu_buffer_rsrc_t wbuf = make_buffer(w, (unsigned)V * (unsigned)D * 2u);
  const __amdgpu_buffer_rsrc_t bbuf = make_buffer(bias ? bias : den, bias ? (unsigned)V * 4u : 0u);
  // a tile's rows of x as a raw buffer: rows past the array (and whole tiles past the
  // last one) read as zeros
  auto x_tile = [&](int64_t tile) {
    const int64_t r0 = min(tile, ntiles) * kProjRows;
    const unsigned n = (unsigned)max((int64_t)0, min((int64_t)kProjRows, rows - r0));
    return make_buffer(x + min(r0, rows - 1) * D, n * (unsigned)D * 2u);
  };

  // stage copy: a stage is 32 k-values = 4 chunks of 16 bytes per row; chunk cc of
  // row r lives in slot 4 r + (cc ^ ((r >> 2) & 3)).  Thread t moves pieces
  // t, t + 256, ... of W and of x (piece p: row p / 4, chunk p % 4).
  // Pieces t + 256 q of a thread are 64 rows apart: same chunk, same swizzle.
  const unsigned piece_src = ((unsigned)(tid >> 2) * (unsigned)D + 8u * (tid & 3)) * 2u;
  const unsigned piece_dst = (unsigned)(4 * (tid >> 2) + ((tid & 3) ^ ((tid >> 4) & 3))) * 16u;
  const unsigned piece_src_step = 64u * (unsigned)D * 2u;
  constexpr unsigned kPieceDstStep = 64u * 4u * 16u;
  // fragments.  MFMA step ks of a stage takes chunk 2 h + ks from lane group h of both
  // operands: W row 128 wn + 32 vt + c, x row 64 wm + 32 rs + c
  unsigned wfrag[2], xfrag[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const unsigned chunk = (unsigned)((2 * h + ks) ^ ((c >> 2) & 3));
    wfrag[ks] = ((unsigned)(4 * (128 * wn + c)) + chunk) * 16u;
    xfrag[ks] = kProjWBytes + ((unsigned)(4 * (64 * wm + c)) + chunk) * 16u;
  }

  const int ksteps = D / kProjK;

  // global loads run two stages ahead of the matrix work
  // Loads past the last stage are issued all the same (W reads as zeros there, x is
  // re-read): with a branch around them the number of loads in flight would not be
  // known at compile time and every wait would have to drain them all.
  int64_t load_tile = tile_first;
  int load_pass = pass_first, load_kk = 0;
  __amdgpu_buffer_rsrc_t xbuf = x_tile(load_tile);
  auto load_stage = [&](ProjStage &st) {
    const unsigned wbase =
        ((unsigned)(load_pass * kProjCols) * (unsigned)D + (unsigned)(load_kk * kProjK)) * 2u;
#pragma unroll
    for (int q = 0; q < kProjWPieces; ++q)
      st.w[q] = __builtin_amdgcn_raw_buffer_load_b128(wbuf, piece_src, wbase + q * piece_src_step, 0);
#pragma unroll
    for (int q = 0; q < kProjXPieces; ++q)
      st.x[q] = __builtin_amdgcn_raw_buffer_load_b128(
          xbuf, piece_src, (unsigned)(load_kk * kProjK) * 2u + q * piece_src_step, 0);
    if (++load_kk == ksteps) {
      load_kk = 0;
      if (++load_pass == pass_end) {
        load_pass = pass_first;
        load_tile += tile_stride;
        xbuf = x_tile(load_tile);
      }
    }
  };
  auto store_stage = [&](const ProjStage &st, int buf) {
    unsigned char *dst = s_stage + buf * kProjStageBytes;
#pragma unroll
    for (int q = 0; q < kProjWPieces; ++q)
      *reinterpret_cast<u32x4 *>(dst + piece_dst + q * kPieceDstStep) = st.w[q];
#pragma unroll
    for (int q = 0; q < kProjXPieces; ++q)
      *reinterpret_cast<u32x4 *>(dst + kProjWBytes + piece_dst + q * kPieceDstStep) = st.x[q];
  };

  f32x16 acc[2][4];
  auto compute_stage = [&](int buf) {
    const unsigned char *src = s_stage + buf * kProjStageBytes;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      u32x4 wf[4], xf[2];
#pragma unroll
      for (int vt = 0; vt < 4; ++vt)
        wf[vt] = *reinterpret_cast<const u32x4 *>(src + vt * (32 * 4 * 16) + wfrag[ks]);
#pragma unroll
      for (int rs = 0; rs < 2; ++rs)
        xf[rs] = *reinterpret_cast<const u32x4 *>(src + rs * (32 * 4 * 16) + xfrag[ks]);
#pragma unroll
      for (int vt = 0; vt < 4; ++vt)
#pragma unroll
        for (int rs = 0; rs < 2; ++rs) acc[rs][vt] = mfma_32x32x16<E>(wf[vt], xf[rs], acc[rs][vt]);
    }
  };

  ProjStage set_a, set_b;
  // vocabulary entries past V start from -inf and stay there (their rows of W read as
  // zeros), so they drop out of the log-sum-exp without a mask in the epilogue
  auto starting_value = [&](int v) -> float {
    const float b = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(bbuf, (unsigned)v * 4u, 0, 0));
    return v < V ? b : OT_NEG_INF;
  };
  s_bias[tid] = starting_value(pass_first * kProjCols + tid);
  load_stage(set_a);
  load_stage(set_b);
  store_stage(set_a, 0);
  load_stage(set_a);
  for (int64_t tile = tile_first; tile < ntiles; tile += tile_stride) {
  const int64_t row0 = tile * kProjRows;
  const unsigned nrows = (unsigned)min((int64_t)kProjRows, rows - row0);
  // stores to rows past the array vanish
  const __amdgpu_buffer_rsrc_t obuf =
      make_buffer(static_cast<char *>(logits) + row0 * V * kOutBytes, nrows * (unsigned)V * kOutBytes);
  float m_run[2] = {OT_NEG_INF, OT_NEG_INF}, s_run[2] = {0.f, 0.f};
  for (int pass = pass_first; pass < pass_end; ++pass) {
    const int n0 = pass * kProjCols + 128 * wn;  // first column of this wave in the pass
    // accumulators start from the bias: tile (rs, vt), register 4 j + i holds vocabulary
    // entry n0 + 32 vt + 8 j + 4 h + i of packed row 64 wm + 32 rs + c.  The pass's
    // starting values come through LDS (written before the previous pass's stores
    // were issued): a global load here would have to wait for those stores as well.
    lds_barrier();
#pragma unroll
    for (int vt = 0; vt < 4; ++vt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 b4 = *reinterpret_cast<const f32x4 *>(&s_bias[128 * wn + 32 * vt + 8 * j + 4 * h]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[0][vt][4 * j + i] = b4[i];
          acc[1][vt][4 * j + i] = b4[i];
        }
      }
    for (int kk = 0; kk < ksteps; kk += 2) {
      // even stage: buffer 0 is complete, buffer 1 is free; set_b holds the next stage
      lds_barrier();
      store_stage(set_b, 1);
      load_stage(set_b);
      compute_stage(0);
      // odd stage
      lds_barrier();
      store_stage(set_a, 0);
      load_stage(set_a);
      compute_stage(1);
    }

    // epilogue of the pass: round, update the row's running (max, sum), store.
    // A tile's values go through a wave-private LDS tile (32 rows x 32 columns) that
    // turns the accumulator layout (one 16-byte piece per lane and row) into whole
    // 128-byte (64-byte for 2-byte logits) pieces of rows per store instruction.
    unsigned char *tile = s_tile + wave * kProjTileBytes;
    // starting values of the next pass (of the next tile after the last one), fetched
    // before this pass's stores are issued
    if (pass_count > 1) s_bias[tid] = starting_value((pass + 1 < pass_end ? pass + 1 : pass_first) * kProjCols + tid);
    constexpr int kTilePitch = OUT_F32 ? kProjTilePitch : kProjTilePitch / 2 + 8;  // 144 / 80 bytes
    constexpr int kLanesPerRow = OUT_F32 ? 8 : 4;        // 16 bytes per lane
    constexpr int kRowsPerStore = kWave / kLanesPerRow;  // 8 or 16
    constexpr int kUnit = 16 / (int)kOutBytes;           // columns per lane: 4 or 8
    const int q = lane % kLanesPerRow, rr = lane / kLanesPerRow;
#pragma unroll
    for (int rs = 0; rs < 2; ++rs) {
#pragma unroll
      for (int vt = 0; vt < 4; ++vt) {
        // register 4 j + i: column n0 + 32 vt + 8 j + 4 h + i, row c of the tile
        float tmax = OT_NEG_INF;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float y[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) y[i] = acc[rs][vt][4 * j + i];
          if (OUT_F32) {
            const f32x4 t = {y[0], y[1], y[2], y[3]};
            *reinterpret_cast<f32x4 *>(tile + c * kTilePitch + (8 * j + 4 * h) * 4) = t;
          } else {
            const unsigned short b0 = from_float<E>(y[0]), b1 = from_float<E>(y[1]);
            const unsigned short b2 = from_float<E>(y[2]), b3 = from_float<E>(y[3]);
            const u32x2 t = {(unsigned)b0 | ((unsigned)b1 << 16), (unsigned)b2 | ((unsigned)b3 << 16)};
            *reinterpret_cast<u32x2 *>(tile + c * kTilePitch + (8 * j + 4 * h) * 2) = t;
            y[0] = to_float<E>(b0);
            y[1] = to_float<E>(b1);
            y[2] = to_float<E>(b2);
            y[3] = to_float<E>(b3);
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            acc[rs][vt][4 * j + i] = y[i];
            tmax = fmaxf(tmax, y[i]);
          }
        }
        // running (max, sum) of the row over this lane's share of the columns
        const float nm = fmaxf(m_run[rs], tmax);
        const float ref = __builtin_isinf(nm) ? 0.f : nm;
        const float oldref = __builtin_isinf(m_run[rs]) ? 0.f : m_run[rs];
        float sum = (s_run[rs] == 0.f) ? 0.f : s_run[rs] * exp_fast(oldref - ref);
        // exp(y - ref) = 2^(y * log2(e) - ref * log2(e)): one fused multiply-add per term
        constexpr float kLog2e = 1.44269502162933349609375f;
        const float shift = -ref * kLog2e;
#pragma unroll
        for (int e = 0; e < 16; ++e)
          sum += __builtin_amdgcn_exp2f(__builtin_fmaf(acc[rs][vt][e], kLog2e, shift));
        s_run[rs] = sum;
        m_run[rs] = nm;
        // the tile's rows leave as contiguous pieces
#pragma unroll
        for (int it = 0; it < 32 / kRowsPerStore; ++it) {
          const int trow = it * kRowsPerStore + rr;
          const u32x4 t = *reinterpret_cast<const u32x4 *>(tile + trow * kTilePitch + q * 16);
          const int col = n0 + 32 * vt + q * kUnit;
          const unsigned off =
              ((unsigned)(64 * wm + 32 * rs + trow) * (unsigned)V + (unsigned)col) * kOutBytes;
          if (SV == kUnit) {
            if (col < V) __builtin_amdgcn_raw_buffer_store_b128(t, obuf, off, 0, kProjStoreAux);
          } else if (SV * kOutBytes == 8) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
              const u32x2 t2 = {t[2 * p], t[2 * p + 1]};
              if (col + p * SV < V) __builtin_amdgcn_raw_buffer_store_b64(t2, obuf, off + 8u * p, 0, kProjStoreAux);
            }
          } else if (SV * kOutBytes == 4) {
#pragma unroll
            for (int p = 0; p < 4; ++p)
              if (col + p * SV < V) __builtin_amdgcn_raw_buffer_store_b32(t[p], obuf, off + 4u * p, 0, 0);
          } else {  // single 2-byte elements
#pragma unroll
            for (int p = 0; p < 8; ++p)
              if (col + p < V)
                __builtin_amdgcn_raw_buffer_store_b16(
                    (unsigned short)((p & 1) ? (t[p / 2] >> 16) : (t[p / 2] & 0xffffu)), obuf,
                    off + 2u * p, 0, 0);
          }
        }
      }
    }
  }

  // a row's shares meet: the two lanes (c, c + 32) of each of its 2 waves
  auto merge = [](float m1, float s1, float m2, float s2, float &m, float &sum) {
    m = fmaxf(m1, m2);
    const float ref = __builtin_isinf(m) ? 0.f : m;
    const float r1 = __builtin_isinf(m1) ? 0.f : m1, r2 = __builtin_isinf(m2) ? 0.f : m2;
    sum = ((s1 == 0.f) ? 0.f : s1 * exp_fast(r1 - ref)) + ((s2 == 0.f) ? 0.f : s2 * exp_fast(r2 - ref));
  };
#pragma unroll
  for (int rs = 0; rs < 2; ++rs) {
    const float m2 = __shfl_xor(m_run[rs], 32, kWave), s2 = __shfl_xor(s_run[rs], 32, kWave);
    float m, sum;
    merge(m_run[rs], s_run[rs], m2, s2, m, sum);
    if (h == 0) s_part[wn][64 * wm + 32 * rs + c] = make_float2(m, sum);
  }
  lds_barrier();  // LDS only: the tile's stores stay in flight
  if (tid < kProjRows && (unsigned)tid < nrows) {
    float m = s_part[0][tid].x, sum = s_part[0][tid].y;
    merge(m, sum, s_part[1][tid].x, s_part[1][tid].y, m, sum);
    den[row0 + tid] = logf(sum) + (__builtin_isinf(m) ? 0.f : m);
  }
  }  // tiles
}

static inline int launch_status() { return (int)hipGetLastError(); }

// den[r] = log-sum-exp of a row's parts (one per pass over the vocabulary), parts in order
__global__ __launch_bounds__(kBlock) void project_den_merge_kernel(const float *__restrict__ parts,
                                                                  int nparts, int64_t rows,
                                                                  float *__restrict__ den) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r >= rows) return;
  float m = OT_NEG_INF;
  for (int k = 0; k < nparts; ++k) m = fmaxf(m, parts[(int64_t)k * rows + r]);
  const float ref = __builtin_isinf(m) ? 0.f : m;
  float sum = 0.f;
  for (int k = 0; k < nparts; ++k) sum += expf(parts[(int64_t)k * rows + r] - ref);
  den[r] = logf(sum) + ref;
}

// Workgroups of a launch, and whether the passes of a tile can be dealt out to workgroups of
// one XCD (`parts`: room for rows * passes floats, or NULL).
template <class E, bool OUT_F32>
static int launch_project(const unsigned short *x, const unsigned short *w, const float *bias,
                          int64_t rows, int32_t D, int32_t V, void *logits, float *den, float *parts,
                          hipStream_t s) {
  // two resident workgroups per compute unit walk over the 128-row tiles
  int device = 0, cus = 0;
  if (hipGetDevice(&device) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
    return OT_E_BAD_ARG;
  const int64_t tiles = (rows + kProjRows - 1) / kProjRows;
  const int npasses = (V + kProjCols - 1) / kProjCols;
  int64_t blocks = tiles < 2 * (int64_t)cus ? tiles : 2 * (int64_t)cus;
  // paired walk: every XCD's share of the resident workgroups splits evenly over the passes
  // and there is at least one tile for every group of them
  const int64_t resident = 2 * (int64_t)cus / 8 * 8;
  const bool paired = parts && npasses > 1 && resident > 0 && (resident / 8) % npasses == 0 &&
                      tiles * npasses >= resident;
  if (paired) blocks = resident;
  float *const den_out = paired ? parts : den;
  const unsigned esize = OUT_F32 ? 4u : 2u;
  int sv = (int)(16u / esize);  // elements per store
  while (sv > 1 && (V % sv != 0 || (reinterpret_cast<uintptr_t>(logits) & (uintptr_t)(sv * esize - 1))))
    sv >>= 1;
#define OT_LAUNCH_PROJ(SV_)                                                                       \
  hipLaunchKernelGGL((joiner_project_kernel<E, OUT_F32, SV_>), dim3((unsigned)blocks), dim3(kProjThreads), \
                     0, s, x, w, bias, rows, D, V, logits, den_out, paired ? 1 : 0)
  switch (sv) {
    case 8: if constexpr (!OUT_F32) { OT_LAUNCH_PROJ(8); } break;
    case 4: OT_LAUNCH_PROJ(4); break;
    case 2: OT_LAUNCH_PROJ(2); break;
    default: OT_LAUNCH_PROJ(1); break;
  }
#undef OT_LAUNCH_PROJ
  if (paired)
    hipLaunchKernelGGL(project_den_merge_kernel, dim3((unsigned)((rows + kBlock - 1) / kBlock)), dim3(kBlock),
                       0, s, parts, npasses, rows, den);
  return launch_status();
}

}  // namespace ot

using namespace ot;

extern "C" {

static int joiner_project_checked(const void *x, const void *weight, const float *bias, int32_t dtype,
                                  int64_t rows, int32_t D, int32_t V, void *logits, int32_t logits_dtype,
                                  float *den, float *parts, void *stream) {
  if (!x || !weight || !logits || !den || rows <= 0 || rows > INT32_MAX || D <= 0 || V <= 0 ||
      (dtype != OT_DTYPE_F16 && dtype != OT_DTYPE_BF16) ||
      (logits_dtype != OT_DTYPE_F32 && logits_dtype != dtype))
    return OT_E_BAD_ARG;
  // two stages of 32 k-values per turn of the main loop; offsets inside a workgroup's
  // rows and inside W are 32-bit
  if (D % (2 * kProjK) != 0 || ((int64_t)V + 2 * kProjCols) * D * 2 > (int64_t)UINT32_MAX ||
      (int64_t)kProjRows * V * 4 > (int64_t)UINT32_MAX || (int64_t)kProjRows * D * 2 > (int64_t)UINT32_MAX)
    return OT_E_BAD_ARG;
  if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(weight) & 15) ||
      (reinterpret_cast<uintptr_t>(bias) & 15) || (reinterpret_cast<uintptr_t>(den) & 3) ||
      (reinterpret_cast<uintptr_t>(parts) & 3) ||
      (reinterpret_cast<uintptr_t>(logits) & (logits_dtype == OT_DTYPE_F32 ? 3 : 1)))
    return OT_E_MISALIGNED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned short *xp = static_cast<const unsigned short *>(x);
  const unsigned short *wp = static_cast<const unsigned short *>(weight);
  if (dtype == OT_DTYPE_BF16)
    return logits_dtype == OT_DTYPE_F32
               ? launch_project<BF16, true>(xp, wp, bias, rows, D, V, logits, den, parts, s)
               : launch_project<BF16, false>(xp, wp, bias, rows, D, V, logits, den, parts, s);
  return logits_dtype == OT_DTYPE_F32
             ? launch_project<F16, true>(xp, wp, bias, rows, D, V, logits, den, parts, s)
             : launch_project<F16, false>(xp, wp, bias, rows, D, V, logits, den, parts, s);
}

int ot_joiner_project(const void *x, const void *weight, const float *bias, int32_t dtype,
                      int64_t rows, int32_t D, int32_t V, void *logits, int32_t logits_dtype,
                      float *den, void *stream) {
  return joiner_project_checked(x, weight, bias, dtype, rows, D, V, logits, logits_dtype, den, nullptr, stream);
}

size_t ot_joiner_project_workspace_bytes(int64_t rows, int32_t V) {
  if (rows <= 0 || V <= kProjCols) return 0;
  return (size_t)((V + kProjCols - 1) / kProjCols) * (size_t)rows * sizeof(float);
}

int ot_joiner_project_ws(const void *x, const void *weight, const float *bias, int32_t dtype,
                         int64_t rows, int32_t D, int32_t V, void *logits, int32_t logits_dtype,
                         float *den, void *workspace, size_t workspace_bytes, void *stream) {
  float *parts = static_cast<float *>(workspace);
  if (!parts || workspace_bytes < ot_joiner_project_workspace_bytes(rows, V) ||
      ot_joiner_project_workspace_bytes(rows, V) == 0)
    parts = nullptr;
  return joiner_project_checked(x, weight, bias, dtype, rows, D, V, logits, logits_dtype, den, parts, stream);
}

int ot_log_probs_given_den(const void *logits, int32_t dtype, const float *den,
                           const int32_t *targets, const int32_t *target_lengths,
                           const int32_t *row_splits, int32_t N, int32_t targets_cols,
                           int64_t rows, int32_t V, int32_t blank, float *lp, void *stream) {
  if (!logits || !den || !lp || !target_lengths || !row_splits || N <= 0 || rows <= 0 ||
      rows > INT32_MAX || V <= 0 || blank < 0 || blank >= V || targets_cols < 0 ||
      (targets_cols > 0 && !targets) ||
      (dtype != OT_DTYPE_F32 && dtype != OT_DTYPE_F16 && dtype != OT_DTYPE_BF16))
    return OT_E_BAD_ARG;
  if (reinterpret_cast<uintptr_t>(logits) & (dtype == OT_DTYPE_F32 ? 3 : 1)) return OT_E_MISALIGNED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t per_block = (int64_t)kGatherRows * kBlock;
  const dim3 grid((unsigned)((rows + per_block - 1) / per_block));
#define OT_LAUNCH_GGD(T_)                                                                        \
  hipLaunchKernelGGL(gather_rows_kernel<T_>, grid, dim3(kBlock), 0, s, logits, den, targets,      \
                     target_lengths, row_splits, N, targets_cols, (int64_t)0, rows, V, blank, lp)
  if (dtype == OT_DTYPE_F32) OT_LAUNCH_GGD(float);
  else if (dtype == OT_DTYPE_F16) OT_LAUNCH_GGD(F16);
  else OT_LAUNCH_GGD(BF16);
#undef OT_LAUNCH_GGD
  return launch_status();
}

}  // extern "C"
