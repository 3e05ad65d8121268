// Hand-written gfx950 kernels of the transducer-loss path and their C ABI
// (declared in include/ot_transducer.h).
//
// Kernel map (reference file:line each one stands in for):
//   prepare_kernel        row offsets + batch facts      cuda.cu:411-414, transducer-loss.cc:49-62
//   row_ids_kernel        row -> utterance               cuda.cu:40-59 (moderngpu load_balance_search)
//   lse_gather_kernel     per-row logsumexp + gather     cuda.cu:427 + kernels.cu:30-60
//   gather_rows_kernel    gather only (log-softmax in)   kernels.cu:62-88  (ot_device.hip.h)
//   alpha_beta_kernel     lattice DP, both directions    kernels.cu:200-313, 415-519
//   row_coeff_kernel      per-row part of the gradients  kernels.cu:522-779
//   grad_flat_kernel      (rows, V) pass of the gradients kernels.cu:522-779
//   scale_kernel          grad *= loss_grad              transducer_loss.py:162
//   negative_sum_kernel   loss = -sum or -mean of scores transducer_loss.py:145-147
//
// The two kernels that move (rows, V) data are HBM-bound streaming kernels: a
// group of L lanes owns one row, every lane keeps K 128-bit vectors of the row
// in registers, reductions over the row are DPP butterflies inside the group.
// (L, K) are picked from V so that L*K vectors cover a row with little waste
// and a wave has K independent 16-byte loads per lane in flight.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <type_traits>

#include "ot_device.hip.h"
#include "ot_transducer.h"

namespace ot {

// ---------------------------------------------------------------------------
// prepare: exclusive scan of T*(U+1) and the reductions the argument checks need
// ---------------------------------------------------------------------------
constexpr int kPrepThreads = 256;

// One workgroup.  Wave 0 scans the sizes 64 at a time with lane shuffles; all
// waves reduce the lengths and the targets.
__global__ __launch_bounds__(kPrepThreads) void prepare_kernel(
    const int32_t *__restrict__ logit_lengths, const int32_t *__restrict__ target_lengths,
    const int32_t *__restrict__ targets, int N, int targets_cols,
    int32_t *__restrict__ row_splits, int32_t *__restrict__ row_splits_mirror,
    ot_batch_status *__restrict__ status) {
  __shared__ int s_red[6];
  __shared__ long long s_total;
  const int tid = threadIdx.x;
  if (tid == 0) {
    s_red[0] = INT32_MIN;  // targets max
    s_red[1] = INT32_MAX;  // targets min
    s_red[2] = INT32_MIN;  // U max
    s_red[3] = INT32_MAX;  // U min
    s_red[4] = INT32_MIN;  // T max
    s_red[5] = INT32_MAX;  // T min
  }
  __syncthreads();

  if (tid < kWave) {
    long long carry = 0;
    for (int base = 0; base < N; base += kWave) {
      const int i = base + tid;
      long long v = 0;
      if (i < N) v = (long long)logit_lengths[i] * ((long long)target_lengths[i] + 1);
      for (int ofs = 1; ofs < kWave; ofs <<= 1) {
        const long long o = __shfl_up(v, ofs, kWave);
        if (tid >= ofs) v += o;
      }
      // int32 wrap-around like cumsum(int32) of the reference
      if (i < N) {
        const int32_t split = (int32_t)(uint32_t)(unsigned long long)(carry + v);
        row_splits[i + 1] = split;
        if (row_splits_mirror) row_splits_mirror[i + 1] = split;
      }
      carry += __shfl(v, kWave - 1, kWave);
    }
    if (tid == 0) {
      row_splits[0] = 0;
      if (row_splits_mirror) row_splits_mirror[0] = 0;
      s_total = carry;
    }
  }

  int umax = INT32_MIN, umin = INT32_MAX, tmax = INT32_MIN, tmin = INT32_MAX;
  for (int i = tid; i < N; i += kPrepThreads) {
    const int T = logit_lengths[i], U = target_lengths[i];
    umax = max(umax, U); umin = min(umin, U);
    tmax = max(tmax, T); tmin = min(tmin, T);
  }
  // min/max over all N * targets_cols entries: 16-byte loads, several in flight per thread
  int gmax = INT32_MIN, gmin = INT32_MAX;
  const long long ntargets = (long long)N * targets_cols;
  long long done = 0;
  if ((reinterpret_cast<uintptr_t>(targets) & 15) == 0) {
    const int4 *t4 = reinterpret_cast<const int4 *>(targets);
    const long long n4 = ntargets / 4;
#pragma unroll 4
    for (long long i = tid; i < n4; i += kPrepThreads) {
      const int4 v = t4[i];
      gmax = max(max(gmax, v.x), max(max(v.y, v.z), v.w));
      gmin = min(min(gmin, v.x), min(min(v.y, v.z), v.w));
    }
    done = n4 * 4;
  }
  for (long long i = done + tid; i < ntargets; i += kPrepThreads) {
    const int v = targets[i];
    gmax = max(gmax, v); gmin = min(gmin, v);
  }
  for (int ofs = kWave / 2; ofs > 0; ofs >>= 1) {
    gmax = max(gmax, __shfl_xor(gmax, ofs, kWave)); gmin = min(gmin, __shfl_xor(gmin, ofs, kWave));
    umax = max(umax, __shfl_xor(umax, ofs, kWave)); umin = min(umin, __shfl_xor(umin, ofs, kWave));
    tmax = max(tmax, __shfl_xor(tmax, ofs, kWave)); tmin = min(tmin, __shfl_xor(tmin, ofs, kWave));
  }
  if ((tid & (kWave - 1)) == 0) {
    atomicMax(&s_red[0], gmax); atomicMin(&s_red[1], gmin);
    atomicMax(&s_red[2], umax); atomicMin(&s_red[3], umin);
    atomicMax(&s_red[4], tmax); atomicMin(&s_red[5], tmin);
  }
  __syncthreads();
  // The minimum that matters is the one over the entries the kernels read, u < U_b
  // (padding behind them may be -1).  Only a batch whose whole-array minimum is
  // negative needs the second, row-aware pass.
  if (s_red[1] < 0) {
    __syncthreads();
    if (tid == 0) s_red[1] = INT32_MAX;
    __syncthreads();
    int vmin = INT32_MAX;
    for (int b = tid / kWave; b < N; b += kPrepThreads / kWave) {
      const int U = min(target_lengths[b], targets_cols);
      for (int u = tid & (kWave - 1); u < U; u += kWave)
        vmin = min(vmin, targets[(long long)b * targets_cols + u]);
    }
    for (int ofs = kWave / 2; ofs > 0; ofs >>= 1) vmin = min(vmin, __shfl_xor(vmin, ofs, kWave));
    if ((tid & (kWave - 1)) == 0) atomicMin(&s_red[1], vmin);
    __syncthreads();
  }
  if (tid == 0) {
    status->sum_tu = s_total;
    status->targets_max = s_red[0];
    status->targets_min = s_red[1];
    status->target_len_max = s_red[2];
    status->target_len_min = s_red[3];
    status->logit_len_max = s_red[4];
    status->logit_len_min = s_red[5];
  }
}

__global__ void row_ids_kernel(const int32_t *__restrict__ row_splits, int N, int64_t rows,
                               int32_t *__restrict__ row_ids) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r < rows) row_ids[r] = find_utterance(row_splits, N, r);
}

// ---------------------------------------------------------------------------
// per-row log-sum-exp + blank/target gather, one pass over the logits
// ---------------------------------------------------------------------------
// A group of L lanes reduces one row, so a wave reduces G = 64/L rows per pass;
// vector j of a row (VEC floats) is held by lane j mod L of the group in
// register slot j / L.
//
// Memory side: the G rows of a pass are contiguous, so the wave reads them as
// one flat span (lane i takes vectors i, i+64, ...: each load instruction covers
// an aligned, contiguous 1 KiB, which a 2000-byte row cut into 256-byte pieces
// does not) and re-shapes the span into the row-group layout through a
// wave-private LDS buffer.  The loads of the next pass are issued before the
// current pass is reduced.  The blank/target gather then reads LDS, not HBM.
// Rows longer than L*K vectors (L = 64, so flat and row-group layout coincide)
// stream through registers in chunks with a running (max, scaled sum).
template <int VEC, int L, int K>
__global__ __launch_bounds__(kBlock) void lse_gather_kernel(
    const float *__restrict__ logits, const int32_t *__restrict__ targets,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits,
    int N, int targets_cols, int64_t row_begin, int64_t rows, int V, int blank,
    int rows_per_block, float *__restrict__ den, float *__restrict__ lp) {
  constexpr int G = kWave / L;
  constexpr bool kStaged = G > 1;
  __shared__ BlockUtterances bu;
  __shared__ __attribute__((aligned(16))) float s_stage[kStaged ? kWavesPerBlock * kWave * K * VEC : 4];
  __shared__ float s_den[kMaxRowsPerBlock], s_lp[2 * kMaxRowsPerBlock];
  // this launch covers rows [row_begin, rows)
  const int64_t row_first = row_begin + (int64_t)blockIdx.x * rows_per_block;
  const int64_t row_end = min(rows, row_first + rows_per_block);

  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sub = lane % L, g = lane / L;
  const int nvec = V / VEC;  // VEC divides V by construction of the launch
  const bool whole_row = nvec <= L * K;
  float *stage = s_stage + (kStaged ? wave * (kWave * K * VEC) : 0);

  // flat span of the pass that starts at row `base`: registers a[].  The
  // workgroup's rows are one raw buffer, so the tail of the last span (rows past
  // row_end) reads as zeros without a bounds branch.
  const __amdgpu_buffer_rsrc_t block_buf =
      make_buffer(logits + row_first * (int64_t)V, (unsigned)((row_end - row_first) * V * 4));
  Vec<VEC> a[K];
  auto issue_span = [&](int64_t base) {
    const unsigned off0 = (unsigned)(base - row_first) * (unsigned)V * 4u;
#pragma unroll
    for (int k = 0; k < K; ++k) a[k].load_buffer(block_buf, off0 + (unsigned)(k * kWave + lane) * (VEC * 4u));
  };

  int64_t base = row_first + (int64_t)wave * G;
  if (kStaged && whole_row && base < row_end) issue_span(base);
  // the utterance table is only needed for the gather at the end of a pass: its
  // searches run while the first span is in flight
  bu.load(row_splits, N, row_first, row_end - 1);
  const int64_t lattice_rows = row_splits[N];

  for (; base < row_end; base += kWavesPerBlock * G) {
    const int64_t row = base + g;
    const bool active = row < row_end;
    const float *p = logits + (active ? row : row_first) * (int64_t)V;

    float m, s;
    if (whole_row) {
      // whole row in registers: exact max first, then one exp per element
      Vec<VEC> x[K];
      if (kStaged) {
#pragma unroll
        for (int k = 0; k < K; ++k) a[k].store_lds(stage + (k * kWave + lane) * VEC);
        issue_span(base + kWavesPerBlock * G);  // past row_end: all zeros, never used
      }
      float cm = OT_NEG_INF;
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const int j = k * L + sub;
        if (kStaged) {
          // always inside the wave's buffer; slots past the row are masked
          x[k].load_lds(stage + (g * nvec + j) * VEC);
          const bool keep = (j < nvec) & active;
#pragma unroll
          for (int e = 0; e < VEC; ++e) x[k].v[e] = keep ? x[k].v[e] : OT_NEG_INF;
        } else if (j < nvec) {
          x[k].load(p + (int64_t)j * VEC);
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) x[k].v[e] = OT_NEG_INF;
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) cm = fmaxf(cm, x[k].v[e]);
      }
      m = group_allreduce<L>(cm, MaxOp());
      if (__builtin_isinf(m)) m = 0.f;  // as ATen's logsumexp does for an all -inf / +inf row
      float acc = 0.f;
#pragma unroll
      for (int k = 0; k < K; ++k) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc += exp_fast(x[k].v[e] - m);
      }
      s = group_allreduce<L>(acc, SumOp());
    } else {
      // long row: per-lane running (max, scaled sum), merged across lanes at the end
      float lm = OT_NEG_INF, ls = 0.f;
      for (int c0 = 0; c0 < nvec; c0 += L * K) {
        Vec<VEC> x[K];
        float cm = OT_NEG_INF;
#pragma unroll
        for (int k = 0; k < K; ++k) {
          const int j = c0 + k * L + sub;
          if (j < nvec) {
            x[k].load(p + (int64_t)j * VEC);
          } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[k].v[e] = OT_NEG_INF;
          }
#pragma unroll
          for (int e = 0; e < VEC; ++e) cm = fmaxf(cm, x[k].v[e]);
        }
        const float nm = fmaxf(lm, cm);
        const float ref = __builtin_isinf(nm) ? 0.f : nm;
        float acc = (ls == 0.f) ? 0.f : ls * exp_fast((__builtin_isinf(lm) ? 0.f : lm) - ref);
#pragma unroll
        for (int k = 0; k < K; ++k) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc += exp_fast(x[k].v[e] - ref);
        }
        ls = acc;
        lm = nm;
      }
      m = group_allreduce<L>(lm, MaxOp());
      if (__builtin_isinf(m)) m = 0.f;
      const float lref = __builtin_isinf(lm) ? 0.f : lm;
      const float part = (ls == 0.f) ? 0.f : ls * exp_fast(lref - m);
      s = group_allreduce<L>(part, SumOp());
    }
    const float d = logf(s) + m;

    if (active) {
      const int local = (int)(row - row_first);
      if (sub == 0) s_den[local] = d;
      if (sub < 2 && row < lattice_rows) {
        const Cell c = decode_row(bu, row, nullptr, target_lengths);
        int col = blank;
        bool ok = true;
        if (sub == 1) {
          ok = c.u >= 0 && c.u < c.U && c.u < targets_cols;
          if (ok) {
            col = targets[(int64_t)c.b * targets_cols + c.u];
            ok = (unsigned)col < (unsigned)V;
          }
        }
        float x = 0.f;
        if (ok) x = (kStaged && whole_row) ? stage[g * V + col] : p[col];
        s_lp[2 * local + sub] = ok ? x - d : OT_NEG_INF;
      }
    }
  }
  // The workgroup's results leave in two contiguous pieces (whole cache lines for
  // the usual row counts): 4- and 8-byte stores sprinkled over the read stream cost
  // 5 % of the kernel's time at V = 500.
  __syncthreads();
  const int nrows = (int)(row_end - row_first);
  const int nlp = 2 * (int)max((int64_t)0, min((int64_t)nrows, lattice_rows - row_first));
  for (int i = threadIdx.x; i < nrows; i += kBlock) den[row_first + i] = s_den[i];
  for (int i = threadIdx.x; i < nlp; i += kBlock) lp[2 * row_first + i] = s_lp[i];
}

// ---------------------------------------------------------------------------
// alpha / beta lattice DP: one workgroup per (utterance, direction), one thread
// per u.
//
// Every thread walks its column u with a start delay, t = n - delay(u) for
// alpha (mirrored in t and u for beta):
//   standard lattice        delay = u + wave*kLag   (anti-diagonal wavefront)
//   one symbol per frame    delay = wave*kLag       (all arcs advance t: row sweep)
// A thread keeps what it hands to its two successors in registers.  Inside a
// wave the value for the neighbouring u is exactly one step old and travels by
// a DPP wave shift.  Across a wave boundary it is kLag+1 steps old: the edge
// lane writes it to an LDS ring every step and the next wave reads it kLag+1
// steps later, so one barrier per kChunk = kLag steps orders all LDS traffic
// (none at all for a single wave).  The lp values do not depend on the
// recursion and are fetched kChunk steps ahead.
// ---------------------------------------------------------------------------
constexpr int kMaxDpWaves = OT_LATTICE_TILE / kWave;
constexpr int kChunk = 16;  // steps between barriers
constexpr int kLag = kChunk;
constexpr int kRing = 64;   // >= 2*kChunk + 2 slots per wave boundary

typedef float f32x2 __attribute__((ext_vector_type(2)));

// TILED: the workgroup's threads cover the OT_LATTICE_TILE columns that start at u0, and
// the lattice is swept tile by tile (lattice_tiles).  The column next to the tile on the
// side the recursion comes from belongs to a tile that is already complete in `out`; the
// tile's edge lane takes its neighbour values from there, one load per step, fetched a
// chunk at a time like the values that cross a wave boundary.
template <bool BETA, bool OSF, bool MULTI, bool TILED = false>
__device__ __forceinline__ void lattice_sweep(const float *__restrict__ lp, int T, int U,
                                              int64_t row0, float *__restrict__ out,
                                              float *__restrict__ score,
                                              float (*s_ring)[kRing + kChunk], int u0 = 0) {
  static_assert(MULTI || !TILED, "a tiled sweep has several waves");
  const int u = u0 + (int)threadIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int U1 = U + 1;
  // the sweep's columns are [u0, u_top]
  const int u_top = TILED ? min(U, u0 + OT_LATTICE_TILE - 1) : U;
  const int wlast = (u_top - u0) / kWave;  // wave that owns u_top
  const int nsteps = (OSF ? T : T + (u_top - u0)) + (MULTI ? wlast * kLag : 0);
  const bool column = u <= u_top;
  // (unsigned)(t - u) < band  <=>  u <= t && t - u <= T-1-U   (never, if infeasible)
  const unsigned band = (unsigned)(max(T - 1 - U, -1) + 1);

  int delay;
  if (BETA) delay = (OSF ? 0 : u_top - u) + (MULTI ? (wlast - wave) * kLag : 0);
  else delay = (OSF ? 0 : u - u0) + (MULTI ? wave * kLag : 0);
  // does the recursion enter this tile from a column of another tile?
  const bool gsrc = TILED && (BETA ? u_top < U : u0 > 0);

  // This utterance's slice as raw buffers: a cell index outside [0, T*U1)
  // (t < 0, t >= T, or the forced offset of a thread without a column) reads
  // as 0 and is not written.  Byte offsets are carried directly; the high bit
  // that pushes a column-less thread out of range survives the 32-bit adds.
  const unsigned cells = (unsigned)T * (unsigned)U1;
  const __amdgpu_buffer_rsrc_t lp_buf = make_buffer(lp + 2 * row0, cells * 8u);
  const __amdgpu_buffer_rsrc_t out_buf = make_buffer(out + row0, cells * 4u);
  const unsigned oob = column ? 0u : 0x80000000u;
  const int dt = BETA ? -1 : 1;
  const int dcell = BETA ? -U1 : U1;
  int t = BETA ? (T - 1 + delay) : -delay;  // lattice row at step 0
  const int cell0 = t * U1 + u;
  unsigned off_out = (unsigned)cell0 * 4u + oob;                          // this step's cell
  unsigned off_lp = (unsigned)(cell0 + kChunk * dcell) * 8u + oob;        // kChunk steps ahead
  const unsigned d_out = (unsigned)dcell * 4u, d_lp = (unsigned)dcell * 8u;

  auto fetch = [&](unsigned byte_off) -> f32x2 {
    return __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(lp_buf, byte_off, 0, 0));
  };

  // wave whose edge lane feeds this wave, if any
  const int src_wave = BETA ? wave + 1 : wave - 1;
  const bool has_src = MULTI && src_wave >= 0 && src_wave <= wlast;
  const int src_ok = has_src ? src_wave : wave;  // a ring that exists, for the unconditional read
  const int edge_lane = BETA ? 0 : kWave - 1;
  // where this lane's per-step ring writes go: the edge lane publishes, every
  // other lane hits kChunk dummy slots behind the ring
  float *const ring_dst = &s_ring[wave][(lane == edge_lane) ? 0 : kRing];
  const int ring_mask = (lane == edge_lane) ? (kRing - 1) : 0;
  // lane that holds the edge value of step i of a chunk when the chunk starts: the
  // register is rotated by one lane per step towards the lane that consumes it
  // (lane 0 of an alpha wave, lane 63 of a beta wave)
  const int ering_step = BETA ? (kWave - 1 - lane) : lane;

  // alpha: own = alpha(t-1,u)+blank(t-1,u), nb = alpha(t,u)+sym(t,u) handed to u+1
  // beta : own = nb = beta of the cell computed in the previous step
  // The lattice's start cell falls out of the recursion from own = 0:
  //   alpha(0,0) = log_add(0, -inf) = 0,  beta(T-1,U) = log_add(0 + blank, -inf) = blank.
  // No step is masked: before a thread's first cell everything it sees is -inf
  // (out-of-range lp reads give 0, and -inf + 0 = -inf), after its last cell its
  // values only reach threads that are past their last cell too, and all stores
  // outside the lattice are dropped by the buffer bounds.
  float own = (column && u == (BETA ? U : 0)) ? 0.f : OT_NEG_INF;
  float nb = OT_NEG_INF;

  // Ring of kChunk prefetched lp values: slot i is consumed at step n+i and
  // refilled at once for step n+i+kChunk.
  f32x2 q[kChunk];
#pragma unroll
  for (int i = 0; i < kChunk; ++i) q[i] = fetch((unsigned)(cell0 + i * dcell) * 8u + oob);

  for (int n = 0; n < nsteps; n += kChunk) {
    // the kChunk edge values of this chunk were all written before the last
    // barrier: fetch them with one LDS read, one lane each
    float ering = OT_NEG_INF;
    float *ring_wr = nullptr;
    if (MULTI) {
      // read without a branch (any slot of a valid wave's ring is readable), then select:
      // a branch here splits the loop body and costs register copies of the prefetch ring
      const int s = n - 1 - kLag + ering_step;
      const float v = s_ring[src_ok][s & (kRing - 1)];
      ering = (has_src && ering_step < kChunk && s >= 0) ? v : OT_NEG_INF;
      ring_wr = ring_dst + (n & ring_mask);  // n is a multiple of kChunk: no wrap inside a chunk
      if (TILED && gsrc && wave == (BETA ? wlast : 0)) {
        // The tile's edge column (delay 0) is in row tc at step n + ering_step; what the
        // neighbouring column hands over then is, for alpha, alpha + sym of the cell the
        // symbol arc comes from (same row; the row before on the one-symbol-per-frame
        // lattice) and, for beta, beta of the cell the symbol arc leads to.  Rows outside
        // the lattice hand over -inf.
        const int sc = n + ering_step;
        const int tc = BETA ? (T - 1 - sc) : sc;
        const int te = OSF ? (BETA ? tc + 1 : tc - 1) : tc;
        const int ue = BETA ? u_top + 1 : u0 - 1;
        const bool ok = ering_step < kChunk && (unsigned)te < (unsigned)T;
        const unsigned cell = ok ? (unsigned)(te * U1 + ue) : 0x10000000u;
        // sc0 sc1: served by the device-wide cache, where the earlier tile's stores are
        float e = __builtin_bit_cast(
            float, __builtin_amdgcn_raw_buffer_load_b32(out_buf, cell * 4u, 0, 17));
        if (!BETA)
          e += __builtin_bit_cast(
              float, __builtin_amdgcn_raw_buffer_load_b32(lp_buf, cell * 8u + 4u, 0, 0));
        ering = ok ? e : OT_NEG_INF;
      }
    }
#pragma unroll
    for (int i = 0; i < kChunk; ++i) {
      const f32x2 l = q[i];
      // the lane without a source lane keeps the fill value: the edge of this step
      const float in = BETA ? wave_shift_down(nb, ering) : wave_shift_up(nb, ering);
      if (MULTI) ering = BETA ? dpp_mov<kDppWaveShr1>(ering) : dpp_mov<kDppWaveShl1>(ering);
      float a = BETA ? log_add(own + l.x, in + l.y) : log_add(own, in);
      if (OSF) a = ((unsigned)(t - u) < band) ? a : OT_NEG_INF;
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, a), out_buf, off_out, 0, 0);
      if (BETA) {
        own = nb = a;
      } else {
        own = a + l.x;
        nb = a + l.y;
      }
      if (MULTI) ring_wr[i] = nb;
      // refill the slot only now that l is dead: issued earlier, the load needs a second
      // register pair and the loop ends in copies that wait for the loads in flight
      q[i] = fetch(off_lp);
      if (OSF) t += dt;
      off_out += d_out;
      off_lp += d_lp;
    }
    if (MULTI) lds_barrier();
  }

  // The utterance's score is read back from what this thread stored itself
  // (alpha: thread U's alpha(T-1,U) plus blank(T-1,U); beta: thread 0's beta(0,0)).
  if (column && u == (BETA ? 0 : U)) {
    __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have completed
    if (BETA) {
      *score = out[row0];
    } else {
      const int64_t last = row0 + (int64_t)cells - 1;
      *score = out[last] + lp[2 * last];
    }
  }
}

// ---------------------------------------------------------------------------
// Standard lattice with three or more waves per workgroup.
//
// On the anti-diagonal wavefront the 64 lanes of a wave touch 64 different rows of
// lp and of alpha/beta in every step: 64 cache lines per load and per store
// instruction, and from three waves on the CU's address unit, not the recursion,
// sets the pace.  Here the lanes of a group of G consecutive columns access the
// SAME row in one instruction, G*8 (lp) or G*4 (alpha/beta) contiguous bytes:
//   - lp: every lane loads its own column's value of a row that lies kk + 18 steps
//     ahead of it, kk = its distance from the group's leading lane (0..G-1); the
//     value waits in a wave-private LDS ring of G rows until the lane gets there;
//   - alpha/beta: every lane parks its result in a second LDS ring and stores the
//     one it computed G-1-kk steps ago, which lies in the row the group's trailing
//     lane has just finished.
// A lane only ever reads LDS slots it wrote itself, in program order, so the
// staging needs no synchronisation; LDS reads are issued two steps before use.
// The recursion, the cross-wave hand-over and the barrier per kChunk steps are
// those of lattice_sweep.  Two compute-free chunks fill the rings first.
// ---------------------------------------------------------------------------
constexpr int kStageLead = kChunk + 2;   // steps between a load and its use, for kk = 0
constexpr int kStageWarmup = 2 * kChunk; // compute-free steps in front

template <bool BETA, int G>
__device__ __forceinline__ void lattice_sweep_staged(const float *__restrict__ lp, int T, int U,
                                                     int64_t row0, float *__restrict__ out,
                                                     float *__restrict__ score,
                                                     float (*s_ring)[kRing + kChunk],
                                                     float *s_stage) {
  static_assert(G >= 2 && G <= kChunk && (G & (G - 1)) == 0, "group size");
  const int u = threadIdx.x;
  const int lane = u & (kWave - 1), wave = u / kWave;
  const int nwaves = blockDim.x / kWave;
  const int U1 = U + 1;
  const int wlast = U / kWave;
  const int nsteps = T + U + wlast * kLag;
  const bool column = u < U1;
  const int delay = BETA ? (U - u) + (wlast - wave) * kLag : u + wave * kLag;
  const int kk = BETA ? (G - 1 - (lane & (G - 1))) : (lane & (G - 1));
  const int jj = (G - 1) - kk;

  const unsigned cells = (unsigned)T * (unsigned)U1;
  const __amdgpu_buffer_rsrc_t lp_buf = make_buffer(lp + 2 * row0, cells * 8u);
  const __amdgpu_buffer_rsrc_t out_buf = make_buffer(out + row0, cells * 4u);
  const unsigned oob = column ? 0u : 0x80000000u;
  const int dcell = BETA ? -U1 : U1;
  const int t0 = BETA ? (T - 1 + delay) : -delay;  // lattice row at step 0
  const int cell0 = t0 * U1 + u;
  const unsigned d_out = (unsigned)dcell * 4u, d_lp = (unsigned)dcell * 8u;
  // step n loads the lp cell of step n + kChunk + kStageLead + kk - kChunk ... in full:
  // issued at step n, in a register until step n + kChunk, in LDS until step n + kChunk + kk + 2
  unsigned off_lp = (unsigned)(cell0 + (kStageLead + kk - kStageWarmup) * dcell) * 8u + oob;
  // step n stores the cell of step n - 2 - jj
  unsigned off_st = (unsigned)(cell0 - (2 + jj) * dcell) * 4u + oob;

  auto fetch = [&](unsigned byte_off) -> f32x2 {
    return __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(lp_buf, byte_off, 0, 0));
  };

  f32x2 *const lp_ring = reinterpret_cast<f32x2 *>(s_stage) + wave * (G * kWave) + lane;
  float *const out_ring = s_stage + nwaves * (2 * G * kWave) + wave * (G * kWave) + lane;

  const int src_wave = BETA ? wave + 1 : wave - 1;
  const bool has_src = src_wave >= 0 && src_wave <= wlast;
  const int src_ok = has_src ? src_wave : wave;
  const int edge_lane = BETA ? 0 : kWave - 1;
  float *const ring_dst = &s_ring[wave][(lane == edge_lane) ? 0 : kRing];
  const int ring_mask = (lane == edge_lane) ? (kRing - 1) : 0;
  const int ering_step = BETA ? (kWave - 1 - lane) : lane;

  float own = (column && u == (BETA ? U : 0)) ? 0.f : OT_NEG_INF;
  float nb = OT_NEG_INF;

  f32x2 q[kChunk];
#pragma unroll
  for (int i = 0; i < kChunk; ++i)
    q[i] = fetch((unsigned)(cell0 + (i - kChunk + kStageLead + kk - kStageWarmup) * dcell) * 8u + oob);
  f32x2 lpipe[2] = {{0.f, 0.f}, {0.f, 0.f}};
  float spipe[2] = {0.f, 0.f};

  // kChunk steps starting at step n (a multiple of kChunk); LIVE = false only stages lp
  auto chunk = [&](auto live_tag, int n) {
    constexpr bool LIVE = decltype(live_tag)::value;
    float ering = OT_NEG_INF;
    float *ring_wr = nullptr;
    if (LIVE) {
      const int s = n - 1 - kLag + ering_step;
      const float v = s_ring[src_ok][s & (kRing - 1)];
      ering = (has_src && ering_step < kChunk && s >= 0) ? v : OT_NEG_INF;
      ring_wr = ring_dst + (n & ring_mask);
    }
#pragma unroll
    for (int i = 0; i < kChunk; ++i) {
      // lp: register -> LDS slot of the step that uses it; LDS -> register for step i + 2
      lp_ring[((i + kk + 2) & (G - 1)) * kWave] = q[i];
      q[i] = fetch(off_lp);
      off_lp += d_lp;
      const f32x2 l = lpipe[i & 1];
      lpipe[i & 1] = lp_ring[((i + 2) & (G - 1)) * kWave];
      if (LIVE) {
        const float in = BETA ? wave_shift_down(nb, ering) : wave_shift_up(nb, ering);
        ering = BETA ? dpp_mov<kDppWaveShr1>(ering) : dpp_mov<kDppWaveShl1>(ering);
        const float a = BETA ? log_add(own + l.x, in + l.y) : log_add(own, in);
        out_ring[(i & (G - 1)) * kWave] = a;
        const float st = spipe[i & 1];
        spipe[i & 1] = out_ring[((i + kk + 1) & (G - 1)) * kWave];  // slot of step i - jj
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, st), out_buf, off_st, 0, 0);
        off_st += d_out;
        if (BETA) {
          own = nb = a;
        } else {
          own = a + l.x;
          nb = a + l.y;
        }
        ring_wr[i] = nb;
      }
    }
    if (LIVE) lds_barrier();
  };

  for (int n = -kStageWarmup; n < 0; n += kChunk) chunk(std::false_type{}, n);
  // the last cell's store trails its computation by up to G + 1 steps
  for (int n = 0; n < nsteps + G + 1; n += kChunk) chunk(std::true_type{}, n);

  if (column && u == (BETA ? 0 : U)) {
    __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have completed
    if (BETA) {
      *score = out[row0];
    } else {
      const int64_t last = row0 + (int64_t)cells - 1;
      *score = out[last] + lp[2 * last];
    }
  }
}

// A lattice kernel that is launched before the host has seen the batch facts checks
// what its memory safety rests on itself and does nothing otherwise (guard_n = N, or 0
// for a launch after validation): the rows of the batch add up to the size of the
// arrays, every utterance has T >= 1 and 0 <= U < the columns the launch was sized for,
// and the byte offsets of its cells (8 bytes each, rows up to 1300 beyond either end
// included) stay below 2^31.
__device__ __forceinline__ bool lattice_guard_ok(const int32_t *__restrict__ row_splits, int guard_n,
                                                 int64_t guard_rows, int T, int U, int max_u1) {
  if (guard_n <= 0) return true;
  return (int64_t)row_splits[guard_n] == guard_rows && T >= 1 && U >= 0 && U < max_u1 &&
         ((int64_t)T + 1300) * ((int64_t)U + 1) < ((int64_t)1 << 28);
}

template <int G, int THREADS>
__global__ __launch_bounds__(THREADS) void alpha_beta_staged_kernel(
    const float *__restrict__ lp, const int32_t *__restrict__ logit_lengths,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits,
    int utt_begin, float *__restrict__ alpha, float *__restrict__ beta,
    float *__restrict__ scores_alpha, float *__restrict__ scores_beta, int max_u1, int guard_n,
    int64_t guard_rows) {
  __shared__ float s_ring[THREADS / kWave][kRing + kChunk];
  extern __shared__ __attribute__((aligned(16))) float s_stage[];
  const int b = utt_begin + blockIdx.x;
  const int T = logit_lengths[b], U = target_lengths[b];
  if (!lattice_guard_ok(row_splits, guard_n, guard_rows, T, U, max_u1)) return;
  // utterances with more columns than this workgroup has threads belong to the tiled launch
  if (U >= (int)blockDim.x) return;
  // a wave none of whose lanes has a column takes no part (a barrier only waits for the
  // waves of the workgroup that have not ended)
  if ((int)(threadIdx.x / kWave) > U / kWave) return;
  const int64_t row0 = row_splits[b];
  if (blockIdx.y == 0)
    lattice_sweep_staged<false, G>(lp, T, U, row0, alpha, scores_alpha + b, s_ring, s_stage);
  else
    lattice_sweep_staged<true, G>(lp, T, U, row0, beta, scores_beta + b, s_ring, s_stage);
}

// ---------------------------------------------------------------------------
// Lattices of up to kServedWaves * 64 columns: the recursion with memory waves beside it.
//
// The waves that walk the recursion ("compute waves", one lane per column as above)
// execute no global memory instruction at all.  Every 64 columns have two more waves:
//   - a loader, which fetches the lp cells of the steps ahead (kLoadAhead chunks of
//     kChunk steps in flight, in registers) and puts each cell into an LDS ring at
//     [step mod 2*kChunk][lane], i.e. where the compute lane that needs it at that step
//     reads it with a compile-time offset;
//   - a storer, which takes the results of the chunk before out of a second ring of the
//     same shape and writes them to alpha/beta.
// On the anti-diagonal wavefront the 64 cells of a step lie in 64 different rows of the
// arrays, which is what the one-thread-per-column sweep pays for from two waves on (64
// cache lines per load and per store instruction).  A chunk of 16 steps of a wave covers a
// parallelogram of 79 rows with 16 consecutive columns each; loader and storer walk it
// row-wise, four rows of 16 columns per instruction, and the LDS rings do the skewing.
// Their latencies (and those of a busy memory system) stay out of the recursion as long
// as the loader is kLoadAhead chunks ahead; when it is not, it arrives late at the chunk's
// barrier and everyone waits for it.
// One barrier per chunk orders everything: the loader writes chunk c+1's slots while the
// compute wave reads chunk c's, the storer reads chunk c-1's results while chunk c's are
// written to the other half of the ring.
// On the one-symbol-per-frame lattice all lanes of a wave are in the same row in every
// step; the band (cells outside it are -inf) is applied to the lp values by the loader:
//   alpha: the blank arc out of a cell with t - u >= T-1-U leaves the band, so that
//          cell's blank term becomes -inf (the final blank is read from memory, not here);
//   beta : both terms of a cell outside the band become -inf.
// The arithmetic of a step is that of lattice_sweep, bit for bit (natural logarithms,
// log_add with the reference's threshold).  Keeping the values as base-2 logarithms would
// take three instructions out of the step's dependent chain (measured: 57 instead of 64 ns
// per step at two waves), but every rounding then falls differently from the reference's,
// and the gradient of a long lattice ends up five times further from the reference's
// (2.5e-3 instead of 4.9e-4 at 2 x 10^3 nats) although no further from the exact one.
// ---------------------------------------------------------------------------
constexpr int kServedWaves = 4;            // compute waves per workgroup, 3 waves per 64 columns
// chunks of lp in flight per loader (20 loads each, at most 63 may be outstanding); two
// where three waves share a SIMD's registers
constexpr int load_ahead(int compute_waves) { return compute_waves <= 2 ? 3 : 2; }
constexpr int kRingSlots = kChunk + 1;     // slots per half: one per step + a dummy for masked lanes

template <int C>
struct ServedLds {
  float ring[C][kRing + kChunk];                  // values that cross a wave boundary
  f32x2 lp[C][2][kRingSlots][kWave];              // lp cells by (step mod 32, lane)
  float out[C][2][kRingSlots][kWave];             // results by (step mod 32, lane)
};

// Which cell instruction k of a loader / storer lane handles in a chunk: step dn within
// the chunk and compute lane j it belongs to (j outside [0, 64) or a column beyond U: none),
// and the lattice row at chunk 0; rows advance by kChunk per chunk (backwards for beta).
template <bool BETA, bool OSF>
struct ServedCells {
  static constexpr int kInstr = OSF ? kChunk : 20;
  int w, wlast, T, U, lane;
  __device__ __forceinline__ void cell(int k, int &dn, int &j, int &t0) const {
    const int r = lane >> 4, c = lane & 15;
    if (OSF) {
      dn = k;
      j = lane;
      const int tt = k - (BETA ? (wlast - w) : w) * kLag;  // steps since the wave's start
      t0 = BETA ? T - 1 - tt : tt;
    } else if (!BETA) {
      // delay = 64w + j + 16w, t + j = n - 80w
      dn = c;
      j = 64 - 4 * k - r + c;
      t0 = -80 * w - 64 + 4 * k + r;
    } else {
      // mirrored: delay = (U - 64w - j) + 16(wlast - w)
      dn = 15 - c;
      j = 4 * k + r - 15 + c;
      const int tt = -(U - 64 * w) - (wlast - w) * kLag + 4 * k + r;
      t0 = T - 1 - tt;
    }
  }
};

template <bool BETA, bool OSF, int C>
__device__ __forceinline__ void served_sweep(const float *__restrict__ lp, int T, int U,
                                             int64_t row0, float *__restrict__ out,
                                             float *__restrict__ score, ServedLds<C> &lds) {
  const int wid = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int role = wid / C, w = wid - role * C;  // 0 compute, 1 loader, 2 storer
  const int U1 = U + 1;
  const int wlast = U / kWave;
  if (w > wlast) return;  // no columns: a barrier only waits for the waves that have not ended
  const int nsteps = (OSF ? T : T + U) + wlast * kLag;
  const int nchunks = (nsteps + kChunk - 1) / kChunk;
  const int diff = T - 1 - U;  // width of the one-symbol-per-frame band; negative: infeasible
  const unsigned cells = (unsigned)T * (unsigned)U1;
  // Offset of a lane that has no cell.  Offsets move by one chunk of rows per chunk, all
  // strides of an utterance add up to less than 2^31 bytes (lattice_guard_ok), and the
  // arrays are shorter than that: counting up from 2^31 (alpha) or down from 2^32 - 1
  // (beta) never reaches them.  Rows before the first or behind the last wrap around to
  // offsets beyond the arrays in the same way.
  constexpr unsigned kOob = BETA ? 0xFFFFFFFFu : 0x80000000u;
  constexpr int kLoadAhead = load_ahead(C);

  if (role == 0) {
    // ---- the recursion: LDS in, LDS out ----
    const int u = w * kWave + lane;
    const bool column = u <= U;
    const int src_wave = BETA ? w + 1 : w - 1;
    const bool has_src = C > 1 && src_wave >= 0 && src_wave <= wlast;
    const int src_ok = has_src ? src_wave : w;
    const int edge_lane = BETA ? 0 : kWave - 1;
    float *const ring_dst = &lds.ring[w][(lane == edge_lane) ? 0 : kRing];
    const int ring_mask = (lane == edge_lane) ? (kRing - 1) : 0;
    const int ering_step = BETA ? (kWave - 1 - lane) : lane;
    float own = (column && u == (BETA ? U : 0) && !(OSF && diff < 0)) ? 0.f : OT_NEG_INF;
    float nb = OT_NEG_INF;
    lds_barrier();  // chunk 0 of lp is in the ring
    for (int c = 0; c < nchunks; ++c) {
      const int n = c * kChunk, half = c & 1;
      const f32x2 *const lp_rd = &lds.lp[w][half][0][lane];
      float *const out_wr = &lds.out[w][half][0][lane];
      float ering = OT_NEG_INF;
      float *ring_wr = nullptr;
      if (C > 1) {
        const int s = n - 1 - kLag + ering_step;
        const float v = lds.ring[src_ok][s & (kRing - 1)];
        ering = (has_src && ering_step < kChunk && s >= 0) ? v : OT_NEG_INF;
        ring_wr = ring_dst + (n & ring_mask);
      }
      f32x2 q[kChunk];
#pragma unroll
      for (int i = 0; i < kChunk; ++i) q[i] = lp_rd[i * kWave];
#pragma unroll
      for (int i = 0; i < kChunk; ++i) {
        const f32x2 l = q[i];
        const float in = BETA ? wave_shift_down(nb, ering) : wave_shift_up(nb, ering);
        if (C > 1) ering = BETA ? dpp_mov<kDppWaveShr1>(ering) : dpp_mov<kDppWaveShl1>(ering);
        const float a = BETA ? log_add(own + l.x, in + l.y) : log_add(own, in);
        out_wr[i * kWave] = a;
        if (BETA) {
          own = nb = a;
        } else {
          own = a + l.x;
          nb = a + l.y;
        }
        if (C > 1) ring_wr[i] = nb;
      }
      lds_barrier();
    }
    // the utterance's score from the last cell of the recursion, which this lane computed
    // in the last step (alpha: alpha(T-1,U) plus blank(T-1,U); beta: beta(0,0))
    if (column && u == (BETA ? 0 : U)) {
      const int nf = nsteps - 1;
      const float af = lds.out[w][(nf / kChunk) & 1][nf & (kChunk - 1)][lane];
      if (BETA) {
        *score = af;
      } else {
        const int64_t last = row0 + (int64_t)cells - 1;
        *score = af + lp[2 * last];
      }
    }
    return;
  }

  // ---- memory waves: per-lane cell map, fixed over the chunks ----
  using Cells = ServedCells<BETA, OSF>;
  constexpr int KI = Cells::kInstr;
  const Cells map{w, wlast, T, U, lane};
  const int drow = BETA ? -kChunk : kChunk;  // rows per chunk
  if (role == 1) {
    const __amdgpu_buffer_rsrc_t lp_buf = make_buffer(lp + 2 * row0, cells * 8u);
    unsigned off[KI];       // byte offset of the cell in chunk 0 (top bit set: no cell)
    int slot[KI];           // element index in lds.lp[w][0], the dummy slot for no cell
    int tu[KI];             // t - u at chunk 0 (one-symbol-per-frame band)
#pragma unroll
    for (int k = 0; k < KI; ++k) {
      int dn, j, t0;
      map.cell(k, dn, j, t0);
      const int u = w * kWave + j;
      const bool lane_ok = j >= 0 && j < kWave;
      // a compute lane without a column (u > U) still reads its slots: it gets zeros, as
      // the out-of-range loads of rows outside the lattice give them, never stale LDS
      off[k] = (lane_ok && u <= U) ? (unsigned)(t0 * U1 + u) * 8u : kOob;
      slot[k] = lane_ok ? dn * kWave + j : kChunk * kWave + lane;
      tu[k] = t0 - u;
    }
    const unsigned dchunk = (unsigned)(drow * U1) * 8u;
    f32x2 reg[kLoadAhead][KI];
    auto issue = [&](f32x2(&r)[KI]) {
#pragma unroll
      for (int k = 0; k < KI; ++k) {
        r[k] = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(lp_buf, off[k], 0, 0));
        off[k] += dchunk;
      }
    };
    // c: the chunk these cells belong to
    auto deposit = [&](const f32x2(&r)[KI], int c) {
      f32x2 *const base = &lds.lp[w][c & 1][0][0];
#pragma unroll
      for (int k = 0; k < KI; ++k) {
        f32x2 v = r[k];
        if (OSF) {
          const int d = tu[k] + c * drow;  // t - u of this cell
          if (BETA) {
            const bool inband = (unsigned)d <= (unsigned)diff && diff >= 0;
            v.x = inband ? v.x : OT_NEG_INF;
            v.y = inband ? v.y : OT_NEG_INF;
          } else {
            v.x = (d >= diff) ? OT_NEG_INF : v.x;
          }
        }
        base[slot[k]] = v;
      }
    };
#pragma unroll
    for (int a = 0; a < kLoadAhead; ++a) issue(reg[a]);
    deposit(reg[0], 0);
    lds_barrier();
    // chunk c: fetch chunk c + kLoadAhead into the registers chunk c has left, hand chunk
    // c + 1 to the ring (its half was read for the last time before the barrier above)
    for (int c = 0; c < nchunks; c += kLoadAhead) {
#pragma unroll
      for (int a = 0; a < kLoadAhead; ++a) {
        if (c + a < nchunks) {
          issue(reg[a]);
          deposit(reg[(a + 1) % kLoadAhead], c + a + 1);
          lds_barrier();
        }
      }
    }
    return;
  }

  {
    const __amdgpu_buffer_rsrc_t out_buf = make_buffer(out + row0, cells * 4u);
    unsigned off[KI];
    int slot[KI];
#pragma unroll
    for (int k = 0; k < KI; ++k) {
      int dn, j, t0;
      map.cell(k, dn, j, t0);
      const int u = w * kWave + j;
      const bool ok = j >= 0 && j < kWave && u <= U;
      off[k] = ok ? (unsigned)(t0 * U1 + u) * 4u : kOob;
      slot[k] = ok ? dn * kWave + j : kChunk * kWave + lane;
    }
    const unsigned dchunk = (unsigned)(drow * U1) * 4u;
    // results of chunk c, once the barrier behind it has been passed
    auto drain = [&](int c) {
      const float *const base = &lds.out[w][c & 1][0][0];
      float v[KI];
#pragma unroll
      for (int k = 0; k < KI; ++k) v[k] = base[slot[k]];
#pragma unroll
      for (int k = 0; k < KI; ++k) {
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v[k]), out_buf, off[k], 0, 0);
        off[k] += dchunk;
      }
    };
    lds_barrier();
    for (int c = 0; c < nchunks; ++c) {
      if (c) drain(c - 1);
      lds_barrier();
    }
    drain(nchunks - 1);
  }
}

template <bool OSF, int C>
__global__ __launch_bounds__(3 * C * kWave) void alpha_beta_served_kernel(
    const float *__restrict__ lp, const int32_t *__restrict__ logit_lengths,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits,
    int utt_begin, float *__restrict__ alpha, float *__restrict__ beta,
    float *__restrict__ scores_alpha, float *__restrict__ scores_beta, int max_u1, int guard_n,
    int64_t guard_rows) {
  __shared__ ServedLds<C> lds;
  const int b = utt_begin + blockIdx.x;
  const int T = logit_lengths[b], U = target_lengths[b];
  if (!lattice_guard_ok(row_splits, guard_n, guard_rows, T, U, max_u1)) return;
  if (T < 1 || U < 0 || U >= C * kWave) return;  // not an utterance of this launch
  const int64_t row0 = row_splits[b];
  if (blockIdx.y == 0)
    served_sweep<false, OSF, C>(lp, T, U, row0, alpha, scores_alpha + b, lds);
  else
    served_sweep<true, OSF, C>(lp, T, U, row0, beta, scores_beta + b, lds);
}

// One sweep per tile of OT_LATTICE_TILE columns, in the order of the recursion (alpha:
// ascending u, beta: descending).  A tile reads the finished neighbouring column from
// `out`, so the workgroup's stores are made visible and all its waves meet between tiles.
template <bool BETA, bool OSF>
__device__ __forceinline__ void lattice_tiles(const float *__restrict__ lp, int T, int U,
                                              int64_t row0, float *__restrict__ out,
                                              float *__restrict__ score,
                                              float (*s_ring)[kRing + kChunk]) {
  const int ntiles = U / OT_LATTICE_TILE + 1;
  for (int k = 0; k < ntiles; ++k) {
    if (k) {
      __threadfence();
      __syncthreads();
    }
    const int tile = BETA ? ntiles - 1 - k : k;
    lattice_sweep<BETA, OSF, true, true>(lp, T, U, row0, out, score, s_ring,
                                         tile * OT_LATTICE_TILE);
  }
}

template <bool OSF, bool MULTI, bool TILED>
__global__ __launch_bounds__(OT_LATTICE_TILE) void alpha_beta_kernel(
    const float *__restrict__ lp, const int32_t *__restrict__ logit_lengths,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits,
    int utt_begin, float *__restrict__ alpha, float *__restrict__ beta,
    float *__restrict__ scores_alpha, float *__restrict__ scores_beta, int max_u1, int guard_n,
    int64_t guard_rows) {
  __shared__ float s_ring[MULTI ? kMaxDpWaves : 1][kRing + kChunk];
  const int b = utt_begin + blockIdx.x;
  const int T = logit_lengths[b], U = target_lengths[b];
  if (!lattice_guard_ok(row_splits, guard_n, guard_rows, T, U, max_u1)) return;
  // The tiled launch takes the utterances with more than OT_LATTICE_TILE columns only, the
  // launch in front of it (same grid) all the others.
  if (TILED ? U < OT_LATTICE_TILE : U >= (int)blockDim.x) return;
  // a wave none of whose lanes has a column takes no part (a barrier only waits for the
  // waves of the workgroup that have not ended)
  if (MULTI && !TILED && (int)(threadIdx.x / kWave) > U / kWave) return;
  const int64_t row0 = row_splits[b];
  if (TILED) {
    if (blockIdx.y == 0)
      lattice_tiles<false, OSF>(lp, T, U, row0, alpha, scores_alpha + b, s_ring);
    else
      lattice_tiles<true, OSF>(lp, T, U, row0, beta, scores_beta + b, s_ring);
  } else if (blockIdx.y == 0) {
    lattice_sweep<false, OSF, MULTI>(lp, T, U, row0, alpha, scores_alpha + b, s_ring);
  } else {
    lattice_sweep<true, OSF, MULTI>(lp, T, U, row0, beta, scores_beta + b, s_ring);
  }
}

// ---------------------------------------------------------------------------
// gradient: a per-row coefficient pass, then one flat streaming pass
// ---------------------------------------------------------------------------
// Everything a row's gradient needs besides its V values, 24 bytes per row:
//   logits input       f = {c, bt, e1, e2}:  grad[v] = exp((x[v] + c) + bt)
//                      minus exp((x[v] + c) + e1) at column col1 and
//                      minus exp((x[v] + c) + e2) at column col2,
//                      with c = (alpha + loss) - den, bt = beta(t, u)
//   log-softmax input  f = {v1, v2, 0, 0}: grad is v1 at col1, v2 at col2, else 0
// e1/e2 are the beta of the node the blank / symbol arc leads to (0 for the
// final blank, which leaves the lattice).  The reference's branch order (blank
// tests before the target test, cpu.cc:514-523) decides which arc owns the
// column when a target equals blank.  col1 == kZeroRow marks an all-zero row
// (outside the one-symbol-per-frame band, or likelihood not finite).

// *loss = -scale * sum(scores) by one whole workgroup of kBlock threads, always in
// the same order: thread i adds scores[i], scores[i + 256], ..., then the lanes of a
// wave, then the four waves.
__device__ __forceinline__ void negative_sum_block(const float *__restrict__ scores, int n,
                                                   float scale, float *__restrict__ loss) {
  __shared__ float s_part[kWavesPerBlock];
  float acc = 0.f;
  for (int i = threadIdx.x; i < n; i += kBlock) acc += scores[i];
  acc = group_allreduce<kWave>(acc, SumOp());
  if ((threadIdx.x & (kWave - 1)) == 0) s_part[threadIdx.x / kWave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) t += s_part[w];
    *loss = -(t * scale);
  }
}

template <bool FLS>
__global__ __launch_bounds__(kBlock) void row_coeff_kernel(
    const float *__restrict__ lp, const float *__restrict__ den,
    const float *__restrict__ alpha, const float *__restrict__ beta,
    const int32_t *__restrict__ targets, const int32_t *__restrict__ logit_lengths,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits, int N,
    int targets_cols, int64_t row_begin, int64_t rows, int blank, int osf, float scale,
    float4 *__restrict__ coef_f, int2 *__restrict__ coef_i, const float *__restrict__ scores,
    float loss_scale, float *__restrict__ loss) {
  __shared__ BlockUtterances bu;
  // optionally the reduced loss as well (the launch after the lattice kernel that
  // would otherwise compute it takes longer to start than to run)
  if (loss && blockIdx.x == 0) negative_sum_block(scores, N, loss_scale, loss);
  const int64_t row_first = row_begin + (int64_t)blockIdx.x * kBlock;
  const int64_t row_end = min(rows, row_first + kBlock);
  bu.load(row_splits, N, row_first, row_end - 1);
  const int64_t row = row_first + threadIdx.x;
  if (row >= row_end) return;
  float4 f = make_float4(0.f, 0.f, 0.f, 0.f);
  int2 ci = make_int2(kZeroRow, -1);
  if (row < (int64_t)row_splits[N]) {
    const Cell c = decode_row(bu, row, logit_lengths, target_lengths);
    const int U1 = c.U + 1, diff = c.T - 1 - c.U;
    const float loss = -beta[c.row0];
    const bool inband = !osf || (c.u <= c.t && c.t - c.u <= diff);
    if (inband && __builtin_fabsf(loss) < __builtin_huge_valf()) {
      const float a = alpha[row];
      const float bt = beta[row];
      const float cc = FLS ? a + loss : (a + loss) - den[row];
      const bool last = (c.t == c.T - 1) && (c.u == c.U);
      const bool blank_open = osf ? (c.t - c.u < diff) : (c.t < c.T - 1);
      const bool has_sym = c.u < c.U;
      int tgt = -1;
      if (has_sym && c.u < targets_cols) tgt = targets[(int64_t)c.b * targets_cols + c.u];
      int col1 = -1, col2 = -1;
      float e1 = 0.f, e2 = 0.f;
      if (last) {
        col1 = blank;
      } else if (blank_open) {
        col1 = blank;
        e1 = beta[row + U1];
      }
      if (has_sym && !(col1 >= 0 && tgt == blank)) {
        col2 = tgt;
        e2 = osf ? beta[row + U1 + 1] : beta[row + 1];
      }
      ci = make_int2(col1, col2);
      if (FLS) {
        const float2 l = reinterpret_cast<const float2 *>(lp)[row];
        f.x = col1 >= 0 ? -exp_any((l.x + cc) + e1) * scale : 0.f;
        f.y = col2 >= 0 ? -exp_any((l.y + cc) + e2) * scale : 0.f;
      } else {
        f = make_float4(cc, bt, e1, e2);
      }
    }
  }
  coef_f[row] = f;
  coef_i[row] = ci;
}

// Flat pass over the (rows, V) array in units of VEC floats: unit i belongs to
// row i / nvec.  Consecutive lanes touch consecutive 16-byte units, so every
// wave instruction moves one aligned, contiguous 1 KiB whatever V is; a
// workgroup owns grad_unroll() * grad_block() consecutive units and exists only for them
// (one-shot grid, non-temporal accesses: the measured optimum here both for the
// read-modify-write stream of the logits input and for the write-only stream
// of the log-softmax input).
// Threads per workgroup and 16-byte units per thread, measured per stream on MI355X.
// In-place stream of the logits input: 256 x 1 (2-7 % faster than 256 x 2; 64 x 1 the
// same, 128 x 1, 128 x 2, 64 x 2 and 64 x 4 slower).  Write-only stream of the
// log-softmax input: 64 x 2, one wave per workgroup (6 % faster than 256 x 2, 3 % than
// 128 x 2; 64 x 4, 128 x 4 slower, 128 x 1 and 256 x 1 20 % slower).  The 4-byte units of
// an unaligned array or of a V that is no multiple of 4 keep 256 x 2.
constexpr int grad_unroll(bool from_log_softmax, int vec) {
  return (from_log_softmax || vec == 1) ? 2 : 1;
}
constexpr int grad_block(bool from_log_softmax, int vec) {
  return (from_log_softmax && vec == 4) ? kWave : kBlock;
}

template <int VEC, bool FLS>
__global__ __launch_bounds__(grad_block(FLS, VEC)) void grad_flat_kernel(
    const float *logits, float *grad, const float4 *__restrict__ coef_f,
    const int2 *__restrict__ coef_i, int64_t unit_begin, int64_t nunits, int nvec, float inv_nvec,
    double inv_nvec_d, float scale, const float *__restrict__ device_factor) {
  constexpr int kGradUnroll = grad_unroll(FLS, VEC);
  constexpr int kGradBlock = grad_block(FLS, VEC);
  // optional second factor that lives on the device (the upstream gradient of the loss)
  const float factor = device_factor ? *device_factor : 1.f;
  if (!FLS) scale *= factor;
  // this launch covers units [unit_begin, nunits)
  const int64_t base = unit_begin + (int64_t)blockIdx.x * (kGradUnroll * kGradBlock);
  // base / nvec through a double reciprocal (exact below 2^53) and one correction step
  int64_t row_base = (int64_t)((double)base * inv_nvec_d);
  {
    const int64_t r = base - row_base * nvec;
    if (r < 0) --row_base; else if (r >= nvec) ++row_base;
  }
  const int rem_base = (int)(base - row_base * nvec);
  // the workgroup's units as raw buffers: the tail of the last workgroup needs no branch
  const unsigned span_bytes =
      (unsigned)min((int64_t)(kGradUnroll * kGradBlock), nunits - base) * (VEC * 4u);
  const __amdgpu_buffer_rsrc_t in_buf = make_buffer(FLS ? grad : logits + base * VEC, span_bytes);
  const __amdgpu_buffer_rsrc_t out_buf = make_buffer(grad + base * VEC, span_bytes);

  Vec<VEC> x[kGradUnroll];
  int rows[kGradUnroll], col0[kGradUnroll];
#pragma unroll
  for (int k = 0; k < kGradUnroll; ++k) {
    const int local = k * kGradBlock + (int)threadIdx.x;
    if (!FLS) x[k].load_buffer(in_buf, (unsigned)local * (VEC * 4u));
    // idx < nvec + kGradUnroll*256 is exact in float; one correction step fixes the quotient
    const int idx = rem_base + local;
    int q = (int)((float)idx * inv_nvec);
    if (q * nvec > idx) --q; else if ((q + 1) * nvec <= idx) ++q;
    rows[k] = q;
    col0[k] = (idx - q * nvec) * VEC;
  }
  const int64_t last_row = (nunits - 1) / nvec;
#pragma unroll
  for (int k = 0; k < kGradUnroll; ++k) {
    const int local = k * kGradBlock + (int)threadIdx.x;
    const int64_t row = min(row_base + rows[k], last_row);
    const float4 f = coef_f[row];
    const int2 ci = coef_i[row];
    Vec<VEC> y;
    if (FLS) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) y.v[e] = 0.f;
      const unsigned d1 = (unsigned)(ci.x - col0[k]), d2 = (unsigned)(ci.y - col0[k]);
      if (d1 < (unsigned)VEC || d2 < (unsigned)VEC) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          if (d1 == (unsigned)e) y.v[e] = f.x * factor;
          if (d2 == (unsigned)e) y.v[e] = f.y * factor;
        }
      }
    } else {
      const bool zero = ci.x == kZeroRow;
#pragma unroll
      for (int e = 0; e < VEC; ++e) y.v[e] = zero ? 0.f : exp_any((x[k].v[e] + f.x) + f.y);
      // at most one element of the unit per special column: pick it and evaluate the
      // subtracted exponential once
      const unsigned d1 = (unsigned)(ci.x - col0[k]), d2 = (unsigned)(ci.y - col0[k]);
      if (d1 < (unsigned)VEC) {
        float xe = x[k].v[0];
#pragma unroll
        for (int e = 1; e < VEC; ++e) xe = (d1 == (unsigned)e) ? x[k].v[e] : xe;
        const float sub = exp_any((xe + f.x) + f.z);
#pragma unroll
        for (int e = 0; e < VEC; ++e) y.v[e] = (d1 == (unsigned)e) ? y.v[e] - sub : y.v[e];
      }
      if (d2 < (unsigned)VEC) {
        float xe = x[k].v[0];
#pragma unroll
        for (int e = 1; e < VEC; ++e) xe = (d2 == (unsigned)e) ? x[k].v[e] : xe;
        const float sub = exp_any((xe + f.x) + f.w);
#pragma unroll
        for (int e = 0; e < VEC; ++e) y.v[e] = (d2 == (unsigned)e) ? y.v[e] - sub : y.v[e];
      }
      if (scale != 1.f) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) y.v[e] *= scale;
      }
    }
    y.store_buffer(out_buf, (unsigned)local * (VEC * 4u));
  }
}

__global__ __launch_bounds__(kBlock) void scale_kernel(float *__restrict__ x, int64_t n,
                                                       const float *__restrict__ factor) {
  const float f = *factor;
  if (f == 1.f) return;  // x * 1 == x exactly: nothing to do
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    // spans of kScaleUnroll * 256 16-byte units: all loads of a span, then all
    // stores, non-temporal; the tail of the last span is cut by the buffer bounds
    constexpr int kScaleUnroll = 4;
    constexpr int64_t kSpan = (int64_t)kScaleUnroll * kBlock;
    const int64_t n4 = n / 4;
    for (int64_t base = (int64_t)blockIdx.x * kSpan; base < n4; base += (int64_t)gridDim.x * kSpan) {
      const unsigned bytes = (unsigned)min(kSpan, n4 - base) * 16u;
      const __amdgpu_buffer_rsrc_t buf = make_buffer(x + base * 4, bytes);
      Vec<4> v[kScaleUnroll];
#pragma unroll
      for (int k = 0; k < kScaleUnroll; ++k)
        v[k].load_buffer(buf, (unsigned)(k * kBlock + (int)threadIdx.x) * 16u);
#pragma unroll
      for (int k = 0; k < kScaleUnroll; ++k) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[k].v[e] *= f;
        v[k].store_buffer(buf, (unsigned)(k * kBlock + (int)threadIdx.x) * 16u);
      }
    }
    for (int64_t i = n4 * 4 + tid; i < n; i += stride) x[i] *= f;
  } else {
    for (int64_t i = tid; i < n; i += stride) x[i] *= f;
  }
}

// loss = -scale * sum(scores): one workgroup, fixed summation order
__global__ __launch_bounds__(kBlock) void negative_sum_kernel(const float *__restrict__ scores,
                                                              int n, float scale,
                                                              float *__restrict__ loss) {
  negative_sum_block(scores, n, scale, loss);
}

__global__ __launch_bounds__(kBlock) void copy_kernel(const float4 *__restrict__ src,
                                                      float4 *__restrict__ dst, int64_t n4) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride)
    dst[i] = src[i];
}

// ---------------------------------------------------------------------------
// host side: geometry and dispatch
// ---------------------------------------------------------------------------
// logits bytes one workgroup of the denominator kernel covers
constexpr int64_t kLseBlockBytes = 256 * 1024;
struct RowTiling {
  int vec, L, K, rows_per_block;
};

// Lanes per row L and register vectors per lane K for a row of V floats.
static RowTiling pick_tiling(int V, bool aligned16) {
  RowTiling t;
  t.vec = (aligned16 && V % 4 == 0) ? 4 : 1;
  const int nvec = V / t.vec;
  int L = 8;
  while (L < kWave && L * 8 < nvec) L *= 2;
  int K = 1;
  while (K < 8 && L * K < nvec) K *= 2;
  t.L = L;
  t.K = K;
  // about 256 KiB of logits per workgroup, a whole number of wave passes
  const int pass = kWavesPerBlock * (kWave / L);
  int64_t want = kLseBlockBytes / ((int64_t)V * 4);
  int rpb = (int)((want / pass) * pass);
  if (rpb < pass) rpb = pass;
  if (rpb > kMaxRowsPerBlock) rpb = kMaxRowsPerBlock;
  t.rows_per_block = rpb;
  return t;
}

static inline bool is_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

#define OT_DISPATCH_K(KERNEL, VEC_, L_, K_, ...)                                         \
  switch (K_) {                                                                          \
    case 1: hipLaunchKernelGGL((KERNEL<VEC_, L_, 1>), grid, dim3(kBlock), 0, s, __VA_ARGS__); break; \
    case 2: hipLaunchKernelGGL((KERNEL<VEC_, L_, 2>), grid, dim3(kBlock), 0, s, __VA_ARGS__); break; \
    case 4: hipLaunchKernelGGL((KERNEL<VEC_, L_, 4>), grid, dim3(kBlock), 0, s, __VA_ARGS__); break; \
    default: hipLaunchKernelGGL((KERNEL<VEC_, L_, 8>), grid, dim3(kBlock), 0, s, __VA_ARGS__); break; \
  }
#define OT_DISPATCH_L(KERNEL, VEC_, L_, K_, ...)                           \
  switch (L_) {                                                            \
    case 8: OT_DISPATCH_K(KERNEL, VEC_, 8, K_, __VA_ARGS__) break;         \
    case 16: OT_DISPATCH_K(KERNEL, VEC_, 16, K_, __VA_ARGS__) break;       \
    case 32: OT_DISPATCH_K(KERNEL, VEC_, 32, K_, __VA_ARGS__) break;       \
    default: OT_DISPATCH_K(KERNEL, VEC_, 64, K_, __VA_ARGS__) break;       \
  }
#define OT_DISPATCH(KERNEL, T_, ...)                                       \
  if ((T_).vec == 4) { OT_DISPATCH_L(KERNEL, 4, (T_).L, (T_).K, __VA_ARGS__) } \
  else { OT_DISPATCH_L(KERNEL, 1, (T_).L, (T_).K, __VA_ARGS__) }

static inline int launch_status() { return (int)hipGetLastError(); }

// compute units of the current device (256 on MI355X); 256 if the query fails
static inline int compute_units() {
  int device = 0, cus = 0;
  if (hipGetDevice(&device) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
    return 256;
  return cus;
}

}  // namespace ot

using namespace ot;

extern "C" {

int ot_row_splits(const int32_t *logit_lengths, const int32_t *target_lengths,
                  const int32_t *targets, int32_t N, int32_t targets_cols, int32_t *row_splits,
                  int32_t *row_splits_mirror, ot_batch_status *status, void *stream) {
  if (!logit_lengths || !target_lengths || !row_splits || !status || N <= 0 || targets_cols < 0 ||
      (targets_cols > 0 && !targets))
    return OT_E_BAD_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(prepare_kernel, dim3(1), dim3(kPrepThreads), 0, s, logit_lengths,
                     target_lengths, targets, N, targets_cols, row_splits, row_splits_mirror,
                     status);
  return launch_status();
}

int ot_row_ids(const int32_t *row_splits, int32_t N, int64_t rows, int32_t *row_ids,
               void *stream) {
  if (!row_splits || !row_ids || N <= 0 || rows < 0 || rows > INT32_MAX) return OT_E_BAD_ARG;
  if (rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned blocks = (unsigned)((rows + kBlock - 1) / kBlock);
  hipLaunchKernelGGL(row_ids_kernel, dim3(blocks), dim3(kBlock), 0, s, row_splits, N, rows, row_ids);
  return launch_status();
}

int ot_log_probs_range(const float *logits, const int32_t *targets, const int32_t *target_lengths,
                       const int32_t *row_splits, int32_t N, int32_t targets_cols, int64_t rows,
                       int32_t V, int32_t blank, int32_t from_log_softmax, int64_t row_begin,
                       int64_t row_end, float *den, float *lp, void *stream) {
  if (!logits || !target_lengths || !row_splits || !lp || N <= 0 || rows <= 0 ||
      rows > INT32_MAX || V <= 0 || blank < 0 || blank >= V || targets_cols < 0 ||
      (targets_cols > 0 && !targets) || (!from_log_softmax && !den) || row_begin < 0 ||
      row_end > rows || row_begin > row_end)
    return OT_E_BAD_ARG;
  if (reinterpret_cast<uintptr_t>(logits) & 3) return OT_E_MISALIGNED;
  if (row_begin == row_end) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t count = row_end - row_begin;
  if (from_log_softmax) {
    const int64_t per_block = (int64_t)kGatherRows * kBlock;
    const unsigned blocks = (unsigned)((count + per_block - 1) / per_block);
    hipLaunchKernelGGL(gather_rows_kernel<float>, dim3(blocks), dim3(kBlock), 0, s,
                       static_cast<const void *>(logits), static_cast<const float *>(nullptr),
                       targets, target_lengths, row_splits, N, targets_cols, row_begin, row_end, V,
                       blank, lp);
    return launch_status();
  }
  const RowTiling t = pick_tiling(V, is_aligned16(logits));
  const dim3 grid((unsigned)((count + t.rows_per_block - 1) / t.rows_per_block));
  OT_DISPATCH(lse_gather_kernel, t, logits, targets, target_lengths, row_splits, N, targets_cols,
              row_begin, row_end, V, blank, t.rows_per_block, den, lp)
  return launch_status();
}

int ot_log_probs(const float *logits, const int32_t *targets, const int32_t *target_lengths,
                 const int32_t *row_splits, int32_t N, int32_t targets_cols, int64_t rows,
                 int32_t V, int32_t blank, int32_t from_log_softmax, float *den, float *lp,
                 void *stream) {
  return ot_log_probs_range(logits, targets, target_lengths, row_splits, N, targets_cols, rows, V,
                            blank, from_log_softmax, 0, rows, den, lp, stream);
}

static int launch_alpha_beta(const float *lp, const int32_t *logit_lengths,
                             const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                             int32_t max_u1, int32_t one_sym_per_frame, int32_t utt_begin,
                             int32_t utt_end, float *alpha, float *beta, float *scores_alpha,
                             float *scores_beta, int guard_n, int64_t guard_rows, void *stream) {
  if (!lp || !logit_lengths || !target_lengths || !row_splits || !alpha || !beta ||
      !scores_alpha || !scores_beta || N <= 0 || max_u1 <= 0 || utt_begin < 0 || utt_end > N ||
      utt_begin > utt_end)
    return OT_E_BAD_ARG;
  if (max_u1 > OT_MAX_U1) return OT_E_TOO_LONG;
  if (utt_begin == utt_end) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // One workgroup per (utterance, direction) with a thread per column, up to
  // OT_LATTICE_TILE columns.  A batch with longer utterances gets two launches over the same
  // grid: this one for the utterances that fit (each workgroup looks at its own U), and a
  // second in which a workgroup of OT_LATTICE_TILE threads sweeps its utterance's columns
  // tile by tile, so that one long utterance does not move the whole batch to that kernel.
  const bool tiled = max_u1 > OT_LATTICE_TILE;
  const int threads = tiled ? OT_LATTICE_TILE : ((max_u1 + kWave - 1) / kWave) * kWave;
  const dim3 grid((unsigned)(utt_end - utt_begin), 2), block((unsigned)threads);
  const bool multi = threads > kWave;
  const int nwaves = threads / kWave;
  if (nwaves <= kServedWaves) {
    // up to 256 columns: compute waves beside loader and storer waves
#define OT_LAUNCH_SERVED(OSF_, C_)                                                              \
  hipLaunchKernelGGL((alpha_beta_served_kernel<OSF_, C_>), grid, dim3(3 * C_ * kWave), 0, s,    \
                     lp, logit_lengths, target_lengths, row_splits, utt_begin, alpha, beta,     \
                     scores_alpha, scores_beta, max_u1, guard_n, guard_rows)
#define OT_LAUNCH_SERVED_C(OSF_)                                                                \
  switch (nwaves) {                                                                             \
    case 1: OT_LAUNCH_SERVED(OSF_, 1); break;                                                   \
    case 2: OT_LAUNCH_SERVED(OSF_, 2); break;                                                   \
    case 3: OT_LAUNCH_SERVED(OSF_, 3); break;                                                   \
    default: OT_LAUNCH_SERVED(OSF_, 4); break;                                                  \
  }
    if (one_sym_per_frame) { OT_LAUNCH_SERVED_C(true) } else { OT_LAUNCH_SERVED_C(false) }
#undef OT_LAUNCH_SERVED_C
#undef OT_LAUNCH_SERVED
    return launch_status();
  }
  if (!one_sym_per_frame && nwaves >= 3) {
    // staging rings: (8 + 4) bytes per lane and group row
    const int G = nwaves <= 4 ? 16 : nwaves <= 9 ? 8 : 4;
    const size_t lds = (size_t)nwaves * G * kWave * 12;
#define OT_LAUNCH_DPS(G_, THREADS_)                                                             \
  hipLaunchKernelGGL((alpha_beta_staged_kernel<G_, THREADS_>), grid, block, lds, s, lp,         \
                     logit_lengths, target_lengths, row_splits, utt_begin, alpha, beta,         \
                     scores_alpha, scores_beta, max_u1, guard_n, guard_rows)
    if (G == 16) OT_LAUNCH_DPS(16, 256);
    else if (G == 8) OT_LAUNCH_DPS(8, 576);
    else OT_LAUNCH_DPS(4, 1024);
#undef OT_LAUNCH_DPS
  } else {
#define OT_LAUNCH_DP(OSF_, MULTI_)                                                              \
  hipLaunchKernelGGL((alpha_beta_kernel<OSF_, MULTI_, false>), grid, block, 0, s, lp,           \
                     logit_lengths, target_lengths, row_splits, utt_begin, alpha, beta,         \
                     scores_alpha, scores_beta, max_u1, guard_n, guard_rows)
    if (one_sym_per_frame) {
      if (multi) OT_LAUNCH_DP(true, true); else OT_LAUNCH_DP(true, false);
    } else {
      if (multi) OT_LAUNCH_DP(false, true); else OT_LAUNCH_DP(false, false);
    }
#undef OT_LAUNCH_DP
  }
  int rc = launch_status();
  if (rc || !tiled) return rc;
#define OT_LAUNCH_TILED(OSF_)                                                                   \
  hipLaunchKernelGGL((alpha_beta_kernel<OSF_, true, true>), grid, dim3(OT_LATTICE_TILE), 0, s,  \
                     lp, logit_lengths, target_lengths, row_splits, utt_begin, alpha, beta,     \
                     scores_alpha, scores_beta, max_u1, guard_n, guard_rows)
  if (one_sym_per_frame) OT_LAUNCH_TILED(true); else OT_LAUNCH_TILED(false);
#undef OT_LAUNCH_TILED
  return launch_status();
}

int ot_alpha_beta_range(const float *lp, const int32_t *logit_lengths,
                        const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                        int32_t max_u1, int32_t one_sym_per_frame, int32_t utt_begin,
                        int32_t utt_end, float *alpha, float *beta, float *scores_alpha,
                        float *scores_beta, void *stream) {
  return launch_alpha_beta(lp, logit_lengths, target_lengths, row_splits, N, max_u1,
                           one_sym_per_frame, utt_begin, utt_end, alpha, beta, scores_alpha,
                           scores_beta, 0, 0, stream);
}

int ot_alpha_beta_guarded(const float *lp, const int32_t *logit_lengths,
                          const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                          int32_t max_u1, int32_t one_sym_per_frame, int64_t rows, float *alpha,
                          float *beta, float *scores_alpha, float *scores_beta, void *stream) {
  if (rows <= 0) return OT_E_BAD_ARG;
  return launch_alpha_beta(lp, logit_lengths, target_lengths, row_splits, N, max_u1,
                           one_sym_per_frame, 0, N, alpha, beta, scores_alpha, scores_beta, N, rows,
                           stream);
}

int ot_alpha_beta(const float *lp, const int32_t *logit_lengths, const int32_t *target_lengths,
                  const int32_t *row_splits, int32_t N, int32_t max_u1, int32_t one_sym_per_frame,
                  float *alpha, float *beta, float *scores_alpha, float *scores_beta,
                  void *stream) {
  return ot_alpha_beta_range(lp, logit_lengths, target_lengths, row_splits, N, max_u1,
                             one_sym_per_frame, 0, N, alpha, beta, scores_alpha, scores_beta,
                             stream);
}

static int launch_row_coefficients(const float *lp, const float *den, const float *alpha,
                                   const float *beta, const int32_t *targets,
                                   const int32_t *logit_lengths, const int32_t *target_lengths,
                                   const int32_t *row_splits, int32_t N, int32_t targets_cols,
                                   int64_t rows, int32_t blank, int32_t from_log_softmax,
                                   int32_t one_sym_per_frame, float grad_scale, int64_t row_begin,
                                   int64_t row_end, void *row_scratch, const float *scores,
                                   float loss_scale, float *loss, void *stream) {
  if (!alpha || !beta || !logit_lengths || !target_lengths || !row_splits || !row_scratch ||
      N <= 0 || rows <= 0 || rows > INT32_MAX || blank < 0 || targets_cols < 0 ||
      (targets_cols > 0 && !targets) || (from_log_softmax ? !lp : !den) || row_begin < 0 ||
      row_end > rows || row_begin > row_end || (loss && !scores))
    return OT_E_BAD_ARG;
  if (reinterpret_cast<uintptr_t>(row_scratch) & 15) return OT_E_MISALIGNED;
  if (row_begin == row_end) return loss ? ot_negative_sum(scores, N, loss_scale, loss, stream) : 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float4 *coef_f = static_cast<float4 *>(row_scratch);
  int2 *coef_i = reinterpret_cast<int2 *>(coef_f + rows);
  const dim3 grid((unsigned)((row_end - row_begin + kBlock - 1) / kBlock));
  if (from_log_softmax)
    hipLaunchKernelGGL(row_coeff_kernel<true>, grid, dim3(kBlock), 0, s, lp, den, alpha, beta,
                       targets, logit_lengths, target_lengths, row_splits, N, targets_cols,
                       row_begin, row_end, blank, one_sym_per_frame, grad_scale, coef_f, coef_i,
                       scores, loss_scale, loss);
  else
    hipLaunchKernelGGL(row_coeff_kernel<false>, grid, dim3(kBlock), 0, s, lp, den, alpha, beta,
                       targets, logit_lengths, target_lengths, row_splits, N, targets_cols,
                       row_begin, row_end, blank, one_sym_per_frame, grad_scale, coef_f, coef_i,
                       scores, loss_scale, loss);
  return launch_status();
}

int ot_row_coefficients_range(const float *lp, const float *den, const float *alpha,
                              const float *beta, const int32_t *targets,
                              const int32_t *logit_lengths, const int32_t *target_lengths,
                              const int32_t *row_splits, int32_t N, int32_t targets_cols,
                              int64_t rows, int32_t blank, int32_t from_log_softmax,
                              int32_t one_sym_per_frame, float grad_scale, int64_t row_begin,
                              int64_t row_end, void *row_scratch, void *stream) {
  return launch_row_coefficients(lp, den, alpha, beta, targets, logit_lengths, target_lengths,
                                 row_splits, N, targets_cols, rows, blank, from_log_softmax,
                                 one_sym_per_frame, grad_scale, row_begin, row_end, row_scratch,
                                 nullptr, 0.f, nullptr, stream);
}

int ot_row_coefficients_loss(const float *lp, const float *den, const float *alpha,
                             const float *beta, const int32_t *targets,
                             const int32_t *logit_lengths, const int32_t *target_lengths,
                             const int32_t *row_splits, int32_t N, int32_t targets_cols,
                             int64_t rows, int32_t blank, int32_t from_log_softmax,
                             int32_t one_sym_per_frame, float grad_scale, void *row_scratch,
                             const float *scores, float loss_scale, float *loss, void *stream) {
  if (!scores || !loss) return OT_E_BAD_ARG;
  return launch_row_coefficients(lp, den, alpha, beta, targets, logit_lengths, target_lengths,
                                 row_splits, N, targets_cols, rows, blank, from_log_softmax,
                                 one_sym_per_frame, grad_scale, 0, rows, row_scratch, scores,
                                 loss_scale, loss, stream);
}

int ot_row_coefficients(const float *lp, const float *den, const float *alpha, const float *beta,
                        const int32_t *targets, const int32_t *logit_lengths,
                        const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                        int32_t targets_cols, int64_t rows, int32_t blank,
                        int32_t from_log_softmax, int32_t one_sym_per_frame, float grad_scale,
                        void *row_scratch, void *stream) {
  return ot_row_coefficients_range(lp, den, alpha, beta, targets, logit_lengths, target_lengths,
                                   row_splits, N, targets_cols, rows, blank, from_log_softmax,
                                   one_sym_per_frame, grad_scale, 0, rows, row_scratch, stream);
}

static int launch_gradient_apply(const float *logits, const void *row_scratch, int64_t rows,
                                 int32_t V, int32_t from_log_softmax, float grad_scale,
                                 const float *device_factor, int64_t row_begin, int64_t row_end,
                                 float *grad, void *stream) {
  if (!row_scratch || !grad || rows <= 0 || rows > INT32_MAX || V <= 0 || row_begin < 0 ||
      row_end > rows || row_begin > row_end)
    return OT_E_BAD_ARG;
  if (from_log_softmax ? grad == logits : !logits) return OT_E_BAD_ARG;
  if ((reinterpret_cast<uintptr_t>(grad) & 3) || (reinterpret_cast<uintptr_t>(logits) & 3) ||
      (reinterpret_cast<uintptr_t>(row_scratch) & 15))
    return OT_E_MISALIGNED;
  if (row_begin == row_end) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float4 *coef_f = static_cast<const float4 *>(row_scratch);
  const int2 *coef_i = reinterpret_cast<const int2 *>(coef_f + rows);
  const bool aligned = is_aligned16(grad) && (from_log_softmax || is_aligned16(logits));
  const int vec = (aligned && V % 4 == 0) ? 4 : 1;
  const int nvec = V / vec;
  const int64_t unit_begin = row_begin * nvec, unit_end = row_end * nvec;
  const int gblock = grad_block(from_log_softmax != 0, vec);
  const int64_t per_block = (int64_t)grad_unroll(from_log_softmax != 0, vec) * gblock;
  const int64_t blocks = (unit_end - unit_begin + per_block - 1) / per_block;
  if (blocks > INT32_MAX) return OT_E_BAD_ARG;
  const dim3 grid((unsigned)blocks);
  const float inv_nvec = 1.0f / (float)nvec;
#define OT_LAUNCH_GRAD(VEC_, FLS_)                                                            \
  hipLaunchKernelGGL((grad_flat_kernel<VEC_, FLS_>), grid, dim3(gblock), 0, s, logits, grad,  \
                     coef_f, coef_i, unit_begin, unit_end, nvec, inv_nvec, 1.0 / (double)nvec,       \
                     grad_scale, device_factor)
  if (from_log_softmax) {
    if (vec == 4) OT_LAUNCH_GRAD(4, true); else OT_LAUNCH_GRAD(1, true);
  } else {
    if (vec == 4) OT_LAUNCH_GRAD(4, false); else OT_LAUNCH_GRAD(1, false);
  }
#undef OT_LAUNCH_GRAD
  return launch_status();
}

int ot_gradient_apply_range(const float *logits, const void *row_scratch, int64_t rows, int32_t V,
                            int32_t from_log_softmax, float grad_scale, int64_t row_begin,
                            int64_t row_end, float *grad, void *stream) {
  return launch_gradient_apply(logits, row_scratch, rows, V, from_log_softmax, grad_scale, nullptr,
                               row_begin, row_end, grad, stream);
}

int ot_gradient_apply(const float *logits, const void *row_scratch, int64_t rows, int32_t V,
                      int32_t from_log_softmax, float grad_scale, float *grad, void *stream) {
  return launch_gradient_apply(logits, row_scratch, rows, V, from_log_softmax, grad_scale, nullptr,
                               0, rows, grad, stream);
}

int ot_gradient_apply_device_factor(const float *logits, const void *row_scratch, int64_t rows,
                                    int32_t V, int32_t from_log_softmax, float grad_scale,
                                    const float *device_factor, float *grad, void *stream) {
  if (!device_factor) return OT_E_BAD_ARG;
  return launch_gradient_apply(logits, row_scratch, rows, V, from_log_softmax, grad_scale,
                               device_factor, 0, rows, grad, stream);
}

int ot_gradient(const float *logits, const float *lp, const float *den, const float *alpha,
                const float *beta, const int32_t *targets, const int32_t *logit_lengths,
                const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                int32_t targets_cols, int64_t rows, int32_t V, int32_t blank,
                int32_t from_log_softmax, int32_t one_sym_per_frame, float grad_scale,
                void *row_scratch, float *grad, void *stream) {
  if (V <= 0 || blank >= V) return OT_E_BAD_ARG;
  int rc = ot_row_coefficients(lp, den, alpha, beta, targets, logit_lengths, target_lengths,
                               row_splits, N, targets_cols, rows, blank, from_log_softmax,
                               one_sym_per_frame, grad_scale, row_scratch, stream);
  if (rc) return rc;
  return ot_gradient_apply(logits, row_scratch, rows, V, from_log_softmax, grad_scale, grad, stream);
}

size_t ot_gradient_scratch_bytes(int64_t rows) {
  return rows > 0 ? (size_t)rows * (sizeof(float4) + sizeof(int2)) : 0;
}

int ot_scale_by_device_scalar(float *x, int64_t n, const float *factor, void *stream) {
  if (!x || !factor || n < 0) return OT_E_BAD_ARG;
  if (n == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // One persistent workgroup per compute unit, 16 KB per workgroup and sweep: a sweep of
  // the grid then covers 4 MB, and workgroup g always works on the pieces g + k * 256.
  // Measured on MI355X for the in-place stream: 6.1 / 5.9 / 5.9 TB/s on 1.5 / 3.0 / 3.9 GB
  // against 5.3 / 4.9 / 4.7 with 4096 workgroups (512: within 2 %, 128: 4.8).
  int64_t blocks = (n / 4 + 4 * kBlock - 1) / (4 * kBlock);
  const int64_t cap = compute_units();
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(scale_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, x, n, factor);
  return launch_status();
}

static inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

size_t ot_workspace_bytes(int32_t N, int64_t rows) {
  if (N <= 0 || rows <= 0) return 0;
  size_t b = 0;
  b += align256(((size_t)N + 1) * sizeof(int32_t));  // row_splits
  b += align256((size_t)N * sizeof(float));          // scores_beta
  b += align256((size_t)rows * sizeof(float));       // den
  b += align256((size_t)rows * 2 * sizeof(float));   // lp
  b += align256((size_t)rows * sizeof(float));       // alpha
  b += align256((size_t)rows * sizeof(float));       // beta
  b += align256(ot_gradient_scratch_bytes(rows));    // per-row gradient coefficients
  return b;
}

int ot_transducer_loss(const float *logits, const int32_t *targets, const int32_t *logit_lengths,
                       const int32_t *target_lengths, int32_t N, int32_t targets_cols,
                       int64_t rows, int32_t V, int32_t blank, int32_t from_log_softmax,
                       int32_t one_sym_per_frame, int32_t max_u1, float grad_scale,
                       void *workspace, size_t workspace_bytes, float *scores, float *grad,
                       ot_batch_status *status, void *stream) {
  if (!workspace || !scores || !status || workspace_bytes < ot_workspace_bytes(N, rows) ||
      (reinterpret_cast<uintptr_t>(workspace) & 255))
    return OT_E_BAD_ARG;
  char *w = static_cast<char *>(workspace);
  int32_t *row_splits = reinterpret_cast<int32_t *>(w); w += align256(((size_t)N + 1) * sizeof(int32_t));
  float *scores_beta = reinterpret_cast<float *>(w);    w += align256((size_t)N * sizeof(float));
  float *den = reinterpret_cast<float *>(w);            w += align256((size_t)rows * sizeof(float));
  float *lp = reinterpret_cast<float *>(w);             w += align256((size_t)rows * 2 * sizeof(float));
  float *alpha = reinterpret_cast<float *>(w);          w += align256((size_t)rows * sizeof(float));
  float *beta = reinterpret_cast<float *>(w);           w += align256((size_t)rows * sizeof(float));
  void *row_scratch = w;
  int rc = ot_row_splits(logit_lengths, target_lengths, targets, N, targets_cols, row_splits,
                         nullptr, status, stream);
  if (rc) return rc;
  rc = ot_log_probs(logits, targets, target_lengths, row_splits, N, targets_cols, rows, V, blank,
                    from_log_softmax, den, lp, stream);
  if (rc) return rc;
  rc = ot_alpha_beta(lp, logit_lengths, target_lengths, row_splits, N, max_u1, one_sym_per_frame,
                     alpha, beta, scores, scores_beta, stream);
  if (rc) return rc;
  if (grad)
    rc = ot_gradient(logits, lp, den, alpha, beta, targets, logit_lengths, target_lengths,
                     row_splits, N, targets_cols, rows, V, blank, from_log_softmax,
                     one_sym_per_frame, grad_scale, row_scratch, grad, stream);
  return rc;
}

// ---------------------------------------------------------------------------
// The whole path for callers that cannot allocate: the workspace is a file-scope
// device array.  Its name is a host-side stand-in, not a device address: the
// address on each device is looked up once with hipGetSymbolAddress and only that
// pointer is ever handed to a kernel.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[OT_STATIC_WORKSPACE_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];  // address of `scratch` on each device, once known

// Address of this device's copy of `scratch` (every GPU holds its own).
int static_scratch(void **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return OT_E_BAD_ARG;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return OT_E_BAD_ARG;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}
}  // namespace

int ot_transducer_loss_static(const float *logits, const int32_t *targets,
                              const int32_t *logit_lengths, const int32_t *target_lengths,
                              int32_t N, int32_t targets_cols, int64_t rows, int32_t V,
                              int32_t blank, int32_t from_log_softmax, int32_t one_sym_per_frame,
                              int32_t max_u1, float grad_scale, float *scores, float *grad,
                              ot_batch_status *status, void *stream) {
  if (N <= 0 || rows <= 0) return OT_E_BAD_ARG;
  // sizes first: a batch that does not fit is refused before anything touches the device
  if (rows > INT32_MAX || ot_workspace_bytes(N, rows) > (size_t)OT_STATIC_WORKSPACE_BYTES)
    return OT_E_TOO_LARGE;
  void *ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc) return rc;
  // every slice of the workspace is written in full before it is read (row offsets,
  // denominators, log-probabilities, every lattice cell, every row's coefficients), so
  // what the previous call left in the array needs no clearing
  return ot_transducer_loss(logits, targets, logit_lengths, target_lengths, N, targets_cols, rows,
                            V, blank, from_log_softmax, one_sym_per_frame, max_u1, grad_scale, ws,
                            (size_t)OT_STATIC_WORKSPACE_BYTES, scores, grad, status, stream);
}

int ot_negative_sum(const float *scores, int32_t N, float scale, float *loss, void *stream) {
  if (!scores || !loss || N <= 0) return OT_E_BAD_ARG;
  hipLaunchKernelGGL(negative_sum_kernel, dim3(1), dim3(kBlock), 0, static_cast<hipStream_t>(stream),
                     scores, N, scale, loss);
  return launch_status();
}

int ot_copy_floats(const float *src, float *dst, int64_t n, void *stream) {
  if (!src || !dst || n < 0 || (n & 3) || !is_aligned16(src) || !is_aligned16(dst))
    return OT_E_BAD_ARG;
  if (n == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int64_t blocks = (n / 4 + 4 * kBlock - 1) / (4 * kBlock);
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                     reinterpret_cast<const float4 *>(src), reinterpret_cast<float4 *>(dst), n / 4);
  return launch_status();
}

const char *ot_error_string(int code) {
  switch (code) {
    case 0: return "success";
    case OT_E_BAD_ARG: return "ot: null pointer, non-positive size or out-of-range argument";
    case OT_E_TOO_LONG: return "ot: a length exceeds what the kernels address (OT_MAX_U1 lattice columns)";
    case OT_E_MISALIGNED: return "ot: float buffer is not 4-byte aligned";
    case OT_E_TOO_LARGE:
      return "ot: the batch needs more workspace than OT_STATIC_WORKSPACE_BYTES; use "
             "ot_transducer_loss with a workspace of ot_workspace_bytes(N, rows)";
    default: return code > 0 ? hipGetErrorString(static_cast<hipError_t>(code)) : "ot: unknown error";
  }
}

}  // extern "C"
