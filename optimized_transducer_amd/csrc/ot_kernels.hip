// Hand-written gfx950 kernels of the transducer-loss path and their C ABI
// (declared in include/ot_transducer.h).
//
// Kernel map (reference file:line each one stands in for):
//   prepare_kernel        row offsets + batch facts      cuda.cu:411-414, transducer-loss.cc:49-62
//   row_ids_kernel        row -> utterance               cuda.cu:40-59 (moderngpu load_balance_search)
//   lse_gather_kernel     per-row logsumexp + gather     cuda.cu:427 + kernels.cu:30-60
//   gather_kernel         gather only (log-softmax in)   kernels.cu:62-88
//   alpha_beta_kernel     lattice DP, both directions    kernels.cu:200-313, 415-519
//   grad_logits_kernel    gradient, logits input         kernels.cu:522-651
//   grad_logsoftmax_kernel gradient, log-softmax input   kernels.cu:653-779
//   scale_kernel          grad *= loss_grad              transducer_loss.py:162
//
// The two kernels that move (rows, V) data are HBM-bound streaming kernels: a
// group of L lanes owns one row, every lane keeps K 128-bit vectors of the row
// in registers, reductions over the row are DPP butterflies inside the group.
// (L, K) are picked from V so that L*K vectors cover a row with little waste
// and a wave has K independent 16-byte loads per lane in flight.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ot_device.hip.h"
#include "ot_transducer.h"

namespace ot {

// ---------------------------------------------------------------------------
// prepare: exclusive scan of T*(U+1) and the reductions the argument checks need
// ---------------------------------------------------------------------------
constexpr int kPrepThreads = 1024;

__global__ __launch_bounds__(kPrepThreads) void prepare_kernel(
    const int32_t *__restrict__ logit_lengths, const int32_t *__restrict__ target_lengths,
    const int32_t *__restrict__ targets, int N, int targets_cols,
    int32_t *__restrict__ row_splits, ot_batch_status *__restrict__ status) {
  __shared__ long long s_scan[kPrepThreads];
  __shared__ long long s_carry;
  __shared__ int s_red[6];
  const int tid = threadIdx.x;
  if (tid == 0) {
    s_carry = 0;
    s_red[0] = INT32_MIN;  // targets max
    s_red[1] = INT32_MAX;  // targets min
    s_red[2] = INT32_MIN;  // U max
    s_red[3] = INT32_MAX;  // U min
    s_red[4] = INT32_MIN;  // T max
    s_red[5] = INT32_MAX;  // T min
    row_splits[0] = 0;
  }
  __syncthreads();

  int umax = INT32_MIN, umin = INT32_MAX, tmax = INT32_MIN, tmin = INT32_MAX;
  for (int base = 0; base < N; base += kPrepThreads) {
    const int i = base + tid;
    long long sz = 0;
    if (i < N) {
      const int T = logit_lengths[i], U = target_lengths[i];
      sz = (long long)T * ((long long)U + 1);
      umax = max(umax, U); umin = min(umin, U);
      tmax = max(tmax, T); tmin = min(tmin, T);
    }
    // Hillis-Steele inclusive scan over the chunk
    s_scan[tid] = sz;
    __syncthreads();
    for (int ofs = 1; ofs < kPrepThreads; ofs <<= 1) {
      const long long add = (tid >= ofs) ? s_scan[tid - ofs] : 0;
      __syncthreads();
      s_scan[tid] += add;
      __syncthreads();
    }
    const long long incl = s_carry + s_scan[tid];
    if (i < N) row_splits[i + 1] = (int32_t)(uint32_t)(unsigned long long)incl;  // int32 wrap like cumsum(int32)
    __syncthreads();
    if (tid == kPrepThreads - 1) s_carry = incl;
    __syncthreads();
  }

  int gmax = INT32_MIN, gmin = INT32_MAX;
  const long long ntargets = (long long)N * targets_cols;
  for (long long i = tid; i < ntargets; i += kPrepThreads) {
    const int v = targets[i];
    gmax = max(gmax, v); gmin = min(gmin, v);
  }
  atomicMax(&s_red[0], gmax); atomicMin(&s_red[1], gmin);
  atomicMax(&s_red[2], umax); atomicMin(&s_red[3], umin);
  atomicMax(&s_red[4], tmax); atomicMin(&s_red[5], tmin);
  __syncthreads();
  if (tid == 0) {
    status->sum_tu = s_carry;
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
// Row r of a workgroup's span is handled by lanes [g*L, g*L+L) of one wave
// (g = r mod 64/L).  Vector j of the row (VEC floats) lives in lane j mod L,
// register slot (j / L) mod K, chunk j / (L*K).
template <int VEC, int L, int K>
__global__ __launch_bounds__(kBlock) void lse_gather_kernel(
    const float *__restrict__ logits, const int32_t *__restrict__ targets,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits,
    int N, int targets_cols, int64_t rows, int V, int blank, int rows_per_block,
    float *__restrict__ den, float *__restrict__ lp) {
  constexpr int G = kWave / L;
  __shared__ BlockUtterances bu;
  const int64_t row_first = (int64_t)blockIdx.x * rows_per_block;
  const int64_t row_end = min(rows, row_first + rows_per_block);
  bu.load(row_splits, N, row_first, row_end - 1);
  const int64_t lattice_rows = row_splits[N];

  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sub = lane % L, g = lane / L;
  const int nvec = V / VEC;  // VEC divides V by construction of the launch

  for (int64_t base = row_first + (int64_t)wave * G; base < row_end; base += kWavesPerBlock * G) {
    const int64_t row = base + g;
    const bool active = row < row_end;
    const float *p = logits + (active ? row : row_first) * (int64_t)V;

    float m, s;
    if (nvec <= L * K) {
      // whole row in registers: exact max first, then one exp per element
      Vec<VEC> x[K];
      float cm = OT_NEG_INF;
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const int j = k * L + sub;
        if (j < nvec) {
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
        for (int e = 0; e < VEC; ++e) acc += expf(x[k].v[e] - m);
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
        float acc = (ls == 0.f) ? 0.f : ls * expf((__builtin_isinf(lm) ? 0.f : lm) - ref);
#pragma unroll
        for (int k = 0; k < K; ++k) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc += expf(x[k].v[e] - ref);
        }
        ls = acc;
        lm = nm;
      }
      m = group_allreduce<L>(lm, MaxOp());
      if (__builtin_isinf(m)) m = 0.f;
      const float lref = __builtin_isinf(lm) ? 0.f : lm;
      const float part = (ls == 0.f) ? 0.f : ls * expf(lref - m);
      s = group_allreduce<L>(part, SumOp());
    }
    const float d = logf(s) + m;

    if (active) {
      if (sub == 0) den[row] = d;
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
        lp[2 * row + sub] = ok ? p[col] - d : OT_NEG_INF;
      }
    }
  }
}

// log-softmax input: no denominator, lp is the two gathered values themselves
__global__ __launch_bounds__(kBlock) void gather_kernel(
    const float *__restrict__ logits, const int32_t *__restrict__ targets,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits,
    int N, int targets_cols, int64_t rows, int V, int blank, float *__restrict__ lp) {
  __shared__ BlockUtterances bu;
  const int64_t row_first = (int64_t)blockIdx.x * kBlock;
  const int64_t row_end = min(rows, row_first + kBlock);
  bu.load(row_splits, N, row_first, row_end - 1);
  const int64_t row = row_first + threadIdx.x;
  if (row >= row_end || row >= (int64_t)row_splits[N]) return;
  const Cell c = decode_row(bu, row, nullptr, target_lengths);
  const float *p = logits + row * (int64_t)V;
  float sym = OT_NEG_INF;
  if (c.u >= 0 && c.u < c.U && c.u < targets_cols) {
    const int col = targets[(int64_t)c.b * targets_cols + c.u];
    if ((unsigned)col < (unsigned)V) sym = p[col];
  }
  reinterpret_cast<float2 *>(lp)[row] = make_float2(p[blank], sym);
}

// ---------------------------------------------------------------------------
// alpha / beta lattice DP: one workgroup per (utterance, direction), one thread
// per u.  Standard lattice: anti-diagonal sweep (T+U steps); one-symbol-per-
// frame lattice: every arc advances t, so a row sweep (T steps) suffices.
// A thread keeps what it hands to its two successors in registers; the value
// for the neighbouring u travels by a DPP wave shift, and between waves through
// a double-buffered LDS slot (one barrier per step, none for a single wave).
// ---------------------------------------------------------------------------
constexpr int kMaxDpWaves = OT_MAX_U1 / kWave;

template <bool BETA, bool OSF, bool MULTI>
__device__ __forceinline__ void lattice_sweep(const float2 *__restrict__ lp, int T, int U,
                                              int64_t row0, float *__restrict__ out,
                                              float *__restrict__ score, float (*s_edge)[kMaxDpWaves + 1]) {
  const int u = threadIdx.x;
  const int lane = u & (kWave - 1), wave = u / kWave;
  const int nwaves = blockDim.x / kWave;
  const int U1 = U + 1;
  const int diff = T - 1 - U;
  const int nsteps = OSF ? T : T + U;
  const float2 ninf2 = make_float2(OT_NEG_INF, OT_NEG_INF);
  const float2 *lpu = lp + row0;

  // lattice row of this thread at step n
  auto t_of = [&](int n) -> int {
    if (BETA) return OSF ? (T - 1 - n) : (T - 1 + U - n - u);
    return OSF ? n : (n - u);
  };
  auto fetch = [&](int n) -> float2 {
    const int t = t_of(n);
    const bool valid = (u < U1) & (t >= 0) & (t < T);
    return valid ? lpu[(int64_t)t * U1 + u] : ninf2;
  };

  // alpha: own = alpha(t-1,u)+blank(t-1,u), nb = alpha(t,u)+sym(t,u) handed to u+1
  // beta : own = nb = beta of the cell computed in the previous step
  float own = OT_NEG_INF, nb = OT_NEG_INF;

  auto step = [&](int n, float2 l) {
    const int t = t_of(n);
    const bool valid = (u < U1) & (t >= 0) & (t < T);
    float edge = OT_NEG_INF;
    if (MULTI) {
      const int src = BETA ? wave + 1 : wave - 1;
      if (src >= 0 && src < nwaves) edge = s_edge[(n + 1) & 1][src];
    }
    const float in = BETA ? wave_shift_down(nb, edge) : wave_shift_up(nb, edge);
    float a;
    if (BETA) {
      a = log_add(own + l.x, in + l.y);
      if (t == T - 1 && u == U) a = l.x;
    } else {
      a = log_add(own, in);
      if (n == 0 && u == 0) a = 0.f;
    }
    if (OSF && !(u <= t && t - u <= diff)) a = OT_NEG_INF;
    if (valid) {
      out[row0 + (int64_t)t * U1 + u] = a;
      if (BETA) {
        own = nb = a;
        if (t == 0 && u == 0) *score = a;
      } else {
        own = a + l.x;
        nb = a + l.y;
        if (t == T - 1 && u == U) *score = own;
      }
    } else {
      own = nb = OT_NEG_INF;
    }
    if (MULTI) {
      if (lane == (BETA ? 0 : kWave - 1)) s_edge[n & 1][wave] = nb;
      __syncthreads();
    }
  };

  // lp values are independent of the recursion: keep them four steps ahead
  float2 q0 = fetch(0), q1 = fetch(1), q2 = fetch(2), q3 = fetch(3);
  for (int n = 0; n < nsteps; n += 4) {
    const float2 p0 = fetch(n + 4), p1 = fetch(n + 5), p2 = fetch(n + 6), p3 = fetch(n + 7);
    step(n, q0);
    if (n + 1 < nsteps) step(n + 1, q1);
    if (n + 2 < nsteps) step(n + 2, q2);
    if (n + 3 < nsteps) step(n + 3, q3);
    q0 = p0; q1 = p1; q2 = p2; q3 = p3;
  }
}

template <bool OSF, bool MULTI>
__global__ __launch_bounds__(OT_MAX_U1) void alpha_beta_kernel(
    const float *__restrict__ lp, const int32_t *__restrict__ logit_lengths,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits,
    float *__restrict__ alpha, float *__restrict__ beta, float *__restrict__ scores_alpha,
    float *__restrict__ scores_beta) {
  __shared__ float s_edge[2][kMaxDpWaves + 1];
  const int b = blockIdx.x;
  const int T = logit_lengths[b], U = target_lengths[b];
  const int64_t row0 = row_splits[b];
  if (MULTI) {
    if (threadIdx.x < 2 * (kMaxDpWaves + 1)) (&s_edge[0][0])[threadIdx.x] = OT_NEG_INF;
    __syncthreads();
  }
  const float2 *lp2 = reinterpret_cast<const float2 *>(lp);
  if (blockIdx.y == 0)
    lattice_sweep<false, OSF, MULTI>(lp2, T, U, row0, alpha, scores_alpha + b, s_edge);
  else
    lattice_sweep<true, OSF, MULTI>(lp2, T, U, row0, beta, scores_beta + b, s_edge);
}

// ---------------------------------------------------------------------------
// gradient kernels
// ---------------------------------------------------------------------------
// What a row needs besides its V values.  col1/col2 are the (at most two)
// columns whose entry has a second exponential subtracted; e1/e2 the beta of
// the lattice node that arc leads to (0 for the final blank, which leaves the
// lattice).  Branch order of the reference (blank tests before the target
// test, cpu.cc:514-523) decides which arc wins when a target equals blank.
struct RowGrad {
  float c;      // (alpha + loss) - den          [logits input]   or alpha + loss
  float bt;     // beta(t, u)
  float e1, e2;
  int col1, col2;
  bool zero;    // row outside the band, or the utterance's likelihood is not finite
};

__device__ __forceinline__ RowGrad row_grad(const Cell &c, int64_t row, bool osf, int blank,
                                            const int32_t *__restrict__ targets, int targets_cols,
                                            const float *__restrict__ alpha,
                                            const float *__restrict__ beta,
                                            const float *__restrict__ den) {
  RowGrad r;
  const int U1 = c.U + 1, diff = c.T - 1 - c.U;
  const float loss = -beta[c.row0];
  const bool inband = !osf || (c.u <= c.t && c.t - c.u <= diff);
  r.zero = !inband || !(__builtin_fabsf(loss) < __builtin_huge_valf());
  r.c = 0.f; r.bt = 0.f; r.e1 = 0.f; r.e2 = 0.f; r.col1 = -1; r.col2 = -1;
  if (r.zero) return r;
  const float a = alpha[row];
  r.bt = beta[row];
  r.c = den ? (a + loss) - den[row] : a + loss;
  const bool last = (c.t == c.T - 1) && (c.u == c.U);
  const bool blank_open = osf ? (c.t - c.u < diff) : (c.t < c.T - 1);
  const bool has_sym = c.u < c.U;
  int tgt = -1;
  if (has_sym && c.u < targets_cols) tgt = targets[(int64_t)c.b * targets_cols + c.u];
  if (last) {
    r.col1 = blank; r.e1 = 0.f;
  } else if (blank_open) {
    r.col1 = blank; r.e1 = beta[row + U1];
  }
  if (has_sym && !(r.col1 >= 0 && tgt == blank)) {
    r.col2 = tgt;
    r.e2 = osf ? beta[row + U1 + 1] : beta[row + 1];
  }
  return r;
}

template <int VEC, int L, int K>
__global__ __launch_bounds__(kBlock) void grad_logits_kernel(
    const float *logits, float *grad, const float *__restrict__ den,
    const float *__restrict__ alpha, const float *__restrict__ beta,
    const int32_t *__restrict__ targets, const int32_t *__restrict__ logit_lengths,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits, int N,
    int targets_cols, int64_t rows, int V, int blank, int osf, float scale, int rows_per_block) {
  constexpr int G = kWave / L;
  __shared__ BlockUtterances bu;
  const int64_t row_first = (int64_t)blockIdx.x * rows_per_block;
  const int64_t row_end = min(rows, row_first + rows_per_block);
  bu.load(row_splits, N, row_first, row_end - 1);

  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sub = lane % L, g = lane / L;
  const int nvec = V / VEC;

  for (int64_t base = row_first + (int64_t)wave * G; base < row_end; base += kWavesPerBlock * G) {
    const int64_t row = base + g;
    if (row >= row_end) continue;
    const float *p = logits + row * (int64_t)V;
    float *q = grad + row * (int64_t)V;

    // issue the row's first chunk of loads before the (dependent) scalar lookups
    Vec<VEC> x[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int j = k * L + sub;
      if (j < nvec) x[k].load(p + (int64_t)j * VEC);
    }
    const Cell c = decode_row(bu, row, logit_lengths, target_lengths);
    const RowGrad r = row_grad(c, row, osf != 0, blank, targets, targets_cols, alpha, beta, den);
    const int j1 = r.col1 >= 0 ? r.col1 / VEC : -1, j2 = r.col2 >= 0 ? r.col2 / VEC : -1;

    for (int c0 = 0; c0 < nvec; c0 += L * K) {
      if (c0 > 0) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
          const int j = c0 + k * L + sub;
          if (j < nvec) x[k].load(p + (int64_t)j * VEC);
        }
      }
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const int j = c0 + k * L + sub;
        if (j >= nvec) continue;
        Vec<VEC> y;
        if (r.zero) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) y.v[e] = 0.f;
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) y.v[e] = expf((x[k].v[e] + r.c) + r.bt);
          if (j == j1 || j == j2) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
              const int col = j * VEC + e;
              if (col == r.col1) y.v[e] -= expf((x[k].v[e] + r.c) + r.e1);
              if (col == r.col2) y.v[e] -= expf((x[k].v[e] + r.c) + r.e2);
            }
          }
          if (scale != 1.f) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) y.v[e] *= scale;
          }
        }
        y.store(q + (int64_t)j * VEC);
      }
    }
  }
}

template <int VEC, int L>
__global__ __launch_bounds__(kBlock) void grad_logsoftmax_kernel(
    const float *__restrict__ lp, float *__restrict__ grad, const float *__restrict__ alpha,
    const float *__restrict__ beta, const int32_t *__restrict__ targets,
    const int32_t *__restrict__ logit_lengths, const int32_t *__restrict__ target_lengths,
    const int32_t *__restrict__ row_splits, int N, int targets_cols, int64_t rows, int V,
    int blank, int osf, float scale, int rows_per_block) {
  constexpr int G = kWave / L;
  __shared__ BlockUtterances bu;
  const int64_t row_first = (int64_t)blockIdx.x * rows_per_block;
  const int64_t row_end = min(rows, row_first + rows_per_block);
  bu.load(row_splits, N, row_first, row_end - 1);

  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sub = lane % L, g = lane / L;
  const int nvec = V / VEC;

  for (int64_t base = row_first + (int64_t)wave * G; base < row_end; base += kWavesPerBlock * G) {
    const int64_t row = base + g;
    if (row >= row_end) continue;
    float *q = grad + row * (int64_t)V;
    const Cell c = decode_row(bu, row, logit_lengths, target_lengths);
    const RowGrad r = row_grad(c, row, osf != 0, blank, targets, targets_cols, alpha, beta, nullptr);
    float v1 = 0.f, v2 = 0.f;
    if (!r.zero) {
      const float2 l = reinterpret_cast<const float2 *>(lp)[row];
      if (r.col1 >= 0) v1 = -expf((l.x + r.c) + r.e1) * scale;
      if (r.col2 >= 0) v2 = -expf((l.y + r.c) + r.e2) * scale;
    }
    const int j1 = r.col1 >= 0 ? r.col1 / VEC : -1, j2 = r.col2 >= 0 ? r.col2 / VEC : -1;
    for (int j = sub; j < nvec; j += L) {
      Vec<VEC> y;
#pragma unroll
      for (int e = 0; e < VEC; ++e) y.v[e] = 0.f;
      if (j == j1 || j == j2) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const int col = j * VEC + e;
          if (col == r.col1) y.v[e] = v1;
          if (col == r.col2) y.v[e] = v2;
        }
      }
      y.store(q + (int64_t)j * VEC);
    }
  }
}

__global__ __launch_bounds__(kBlock) void scale_kernel(float *__restrict__ x, int64_t n,
                                                       const float *__restrict__ factor) {
  const float f = *factor;
  if (f == 1.f) return;  // x * 1 == x exactly: nothing to do
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    float4 *x4 = reinterpret_cast<float4 *>(x);
    const int64_t n4 = n / 4;
    for (int64_t i = tid; i < n4; i += stride) {
      float4 v = x4[i];
      v.x *= f; v.y *= f; v.z *= f; v.w *= f;
      x4[i] = v;
    }
    for (int64_t i = n4 * 4 + tid; i < n; i += stride) x[i] *= f;
  } else {
    for (int64_t i = tid; i < n; i += stride) x[i] *= f;
  }
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
  int64_t want = (256 * 1024) / ((int64_t)V * 4);
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

#define OT_DISPATCH_L_ONLY(KERNEL, VEC_, L_, ...)                                                   \
  switch (L_) {                                                                                     \
    case 8: hipLaunchKernelGGL((KERNEL<VEC_, 8>), grid, dim3(kBlock), 0, s, __VA_ARGS__); break;    \
    case 16: hipLaunchKernelGGL((KERNEL<VEC_, 16>), grid, dim3(kBlock), 0, s, __VA_ARGS__); break;  \
    case 32: hipLaunchKernelGGL((KERNEL<VEC_, 32>), grid, dim3(kBlock), 0, s, __VA_ARGS__); break;  \
    default: hipLaunchKernelGGL((KERNEL<VEC_, 64>), grid, dim3(kBlock), 0, s, __VA_ARGS__); break;  \
  }

static inline int launch_status() { return (int)hipGetLastError(); }

}  // namespace ot

using namespace ot;

extern "C" {

int ot_row_splits(const int32_t *logit_lengths, const int32_t *target_lengths,
                  const int32_t *targets, int32_t N, int32_t targets_cols, int32_t *row_splits,
                  ot_batch_status *status, void *stream) {
  if (!logit_lengths || !target_lengths || !row_splits || !status || N <= 0 || targets_cols < 0 ||
      (targets_cols > 0 && !targets))
    return OT_E_BAD_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(prepare_kernel, dim3(1), dim3(kPrepThreads), 0, s, logit_lengths,
                     target_lengths, targets, N, targets_cols, row_splits, status);
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

int ot_log_probs(const float *logits, const int32_t *targets, const int32_t *target_lengths,
                 const int32_t *row_splits, int32_t N, int32_t targets_cols, int64_t rows,
                 int32_t V, int32_t blank, int32_t from_log_softmax, float *den, float *lp,
                 void *stream) {
  if (!logits || !target_lengths || !row_splits || !lp || N <= 0 || rows <= 0 ||
      rows > INT32_MAX || V <= 0 || blank < 0 || blank >= V || targets_cols < 0 ||
      (targets_cols > 0 && !targets) || (!from_log_softmax && !den))
    return OT_E_BAD_ARG;
  if (reinterpret_cast<uintptr_t>(logits) & 3) return OT_E_MISALIGNED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (from_log_softmax) {
    const unsigned blocks = (unsigned)((rows + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(gather_kernel, dim3(blocks), dim3(kBlock), 0, s, logits, targets,
                       target_lengths, row_splits, N, targets_cols, rows, V, blank, lp);
    return launch_status();
  }
  const RowTiling t = pick_tiling(V, is_aligned16(logits));
  const dim3 grid((unsigned)((rows + t.rows_per_block - 1) / t.rows_per_block));
  OT_DISPATCH(lse_gather_kernel, t, logits, targets, target_lengths, row_splits, N, targets_cols,
              rows, V, blank, t.rows_per_block, den, lp)
  return launch_status();
}

int ot_alpha_beta(const float *lp, const int32_t *logit_lengths, const int32_t *target_lengths,
                  const int32_t *row_splits, int32_t N, int32_t max_u1, int32_t one_sym_per_frame,
                  float *alpha, float *beta, float *scores_alpha, float *scores_beta,
                  void *stream) {
  if (!lp || !logit_lengths || !target_lengths || !row_splits || !alpha || !beta ||
      !scores_alpha || !scores_beta || N <= 0 || max_u1 <= 0)
    return OT_E_BAD_ARG;
  if (max_u1 > OT_MAX_U1) return OT_E_TOO_LONG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int threads = ((max_u1 + kWave - 1) / kWave) * kWave;
  const dim3 grid((unsigned)N, 2), block((unsigned)threads);
  const bool multi = threads > kWave;
#define OT_LAUNCH_DP(OSF_, MULTI_)                                                              \
  hipLaunchKernelGGL((alpha_beta_kernel<OSF_, MULTI_>), grid, block, 0, s, lp, logit_lengths,   \
                     target_lengths, row_splits, alpha, beta, scores_alpha, scores_beta)
  if (one_sym_per_frame) {
    if (multi) OT_LAUNCH_DP(true, true); else OT_LAUNCH_DP(true, false);
  } else {
    if (multi) OT_LAUNCH_DP(false, true); else OT_LAUNCH_DP(false, false);
  }
#undef OT_LAUNCH_DP
  return launch_status();
}

int ot_gradient(const float *logits, const float *lp, const float *den, const float *alpha,
                const float *beta, const int32_t *targets, const int32_t *logit_lengths,
                const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                int32_t targets_cols, int64_t rows, int32_t V, int32_t blank,
                int32_t from_log_softmax, int32_t one_sym_per_frame, float grad_scale,
                float *grad, void *stream) {
  if (!alpha || !beta || !logit_lengths || !target_lengths || !row_splits || !grad || N <= 0 ||
      rows <= 0 || rows > INT32_MAX || V <= 0 || blank < 0 || blank >= V || targets_cols < 0 ||
      (targets_cols > 0 && !targets))
    return OT_E_BAD_ARG;
  if (from_log_softmax ? (!lp || grad == logits) : (!logits || !den)) return OT_E_BAD_ARG;
  if ((reinterpret_cast<uintptr_t>(grad) & 3) || (reinterpret_cast<uintptr_t>(logits) & 3))
    return OT_E_MISALIGNED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool aligned = is_aligned16(grad) && (from_log_softmax || is_aligned16(logits));
  const RowTiling t = pick_tiling(V, aligned);
  const dim3 grid((unsigned)((rows + t.rows_per_block - 1) / t.rows_per_block));
  if (from_log_softmax) {
    if (t.vec == 4) {
      OT_DISPATCH_L_ONLY(grad_logsoftmax_kernel, 4, t.L, lp, grad, alpha, beta, targets,
                         logit_lengths, target_lengths, row_splits, N, targets_cols, rows, V,
                         blank, one_sym_per_frame, grad_scale, t.rows_per_block)
    } else {
      OT_DISPATCH_L_ONLY(grad_logsoftmax_kernel, 1, t.L, lp, grad, alpha, beta, targets,
                         logit_lengths, target_lengths, row_splits, N, targets_cols, rows, V,
                         blank, one_sym_per_frame, grad_scale, t.rows_per_block)
    }
  } else {
    OT_DISPATCH(grad_logits_kernel, t, logits, grad, den, alpha, beta, targets, logit_lengths,
                target_lengths, row_splits, N, targets_cols, rows, V, blank, one_sym_per_frame,
                grad_scale, t.rows_per_block)
  }
  return launch_status();
}

int ot_scale_by_device_scalar(float *x, int64_t n, const float *factor, void *stream) {
  if (!x || !factor || n < 0) return OT_E_BAD_ARG;
  if (n == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int64_t blocks = (n / 4 + kBlock - 1) / kBlock;
  if (blocks > 256 * 16) blocks = 256 * 16;
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
  float *beta = reinterpret_cast<float *>(w);
  int rc = ot_row_splits(logit_lengths, target_lengths, targets, N, targets_cols, row_splits,
                         status, stream);
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
                     one_sym_per_frame, grad_scale, grad, stream);
  return rc;
}

int ot_copy_floats(const float *src, float *dst, int64_t n, void *stream) {
  if (!src || !dst || n < 0 || (n & 3) || !is_aligned16(src) || !is_aligned16(dst))
    return OT_E_BAD_ARG;
  if (n == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int64_t blocks = (n / 4 + kBlock - 1) / kBlock;
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                     reinterpret_cast<const float4 *>(src), reinterpret_cast<float4 *>(dst), n / 4);
  return launch_status();
}

const char *ot_error_string(int code) {
  switch (code) {
    case 0: return "success";
    case OT_E_BAD_ARG: return "ot: null pointer, non-positive size or out-of-range argument";
    case OT_E_TOO_LONG: return "ot: max(target_lengths)+1 exceeds OT_MAX_U1";
    case OT_E_MISALIGNED: return "ot: float buffer is not 4-byte aligned";
    default: return code > 0 ? hipGetErrorString(static_cast<hipError_t>(code)) : "ot: unknown error";
  }
}

}  // extern "C"
