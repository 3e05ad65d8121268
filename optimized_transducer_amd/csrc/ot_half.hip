// Half-precision logits (float16 / bfloat16) for the transducer loss: the two
// kernels that touch the (rows, V) array, with float32 arithmetic inside.
//
// The reference accepts float32 logits only (transducer-loss.cc:33); a caller
// whose joiner runs under mixed precision has to cast first.  Reading the
// 2-byte logits directly halves the traffic of both streaming passes.  Every
// per-row quantity (denominators, log-probabilities, alpha, beta, the gradient
// coefficients) stays float32 and goes through the float32 kernels; only
//   lse_gather_half_*_kernel per-row log-sum-exp + blank/target gather (flat: rows
//                            as one stream re-shaped through LDS, for V a multiple
//                            of 4 up to 1024; wide: aligned 16-byte pieces with
//                            masked row ends; plain: any alignment and length)
//   gather_half_kernel       gather only (log-softmax input)
//   grad_flat_half_kernel    (rows, V) gradient pass, in place for logits input
// are specific to the element type.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "ot_device.hip.h"
#include "ot_transducer.h"

namespace ot {

// VEC consecutive elements <-> floats; VEC * 2 bytes per access
template <class E, int VEC> struct HalfIO {
  static_assert(VEC == 1 || VEC == 2 || VEC == 4 || VEC == 8, "elements per access");
  typedef unsigned short raw_t __attribute__((ext_vector_type(VEC)));
  static __device__ __forceinline__ void load(const unsigned short *p, float (&v)[VEC]) {
    raw_t r;
    if (VEC == 1) r[0] = __builtin_nontemporal_load(p);
    else r = __builtin_nontemporal_load(reinterpret_cast<const raw_t *>(p));
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = to_float<E>(r[e]);
  }
  // ordinary load: for row pieces that share cache lines with their neighbours, where
  // the non-temporal hint costs 20 %
  static __device__ __forceinline__ void load_cached(const unsigned short *p, float (&v)[VEC]) {
    raw_t r;
    if (VEC == 1) r[0] = *p;
    else r = *reinterpret_cast<const raw_t *>(p);
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = to_float<E>(r[e]);
  }
  static __device__ __forceinline__ void store(unsigned short *p, const float (&v)[VEC]) {
    raw_t r;
#pragma unroll
    for (int e = 0; e < VEC; ++e) r[e] = from_float<E>(v[e]);
    if (VEC == 1) __builtin_nontemporal_store(r[0], p);
    else __builtin_nontemporal_store(r, reinterpret_cast<raw_t *>(p));
  }
};

// ---------------------------------------------------------------------------
// per-row log-sum-exp + gather: one wave per row, kHalfRowsPerWave rows per wave,
// RB of them in flight at a time
// ---------------------------------------------------------------------------
constexpr int kHalfRowsPerWave = 16;

// Outputs of one wave's rows: dvec holds row r's denominator in lane r.  Lanes
// 0..15 store the denominators as one contiguous piece; lane pair (2r, 2r+1)
// gathers the blank and the target value of row r.
template <class E>
__device__ __forceinline__ void finish_rows(float dvec, int lane, int64_t row_first, int64_t row_end,
                                            const unsigned short *__restrict__ logits,
                                            const int32_t *__restrict__ targets,
                                            const int32_t *__restrict__ target_lengths,
                                            const int32_t *__restrict__ row_splits, int N,
                                            int targets_cols, int V, int blank,
                                            float *__restrict__ den, float *__restrict__ lp) {
  if (lane < kHalfRowsPerWave && row_first + lane < row_end) den[row_first + lane] = dvec;
  const int r = lane >> 1, which = lane & 1;
  const float d = __shfl(dvec, r, kWave);
  const int64_t row = row_first + r;
  const int64_t lattice_rows = row_splits[N];
  if (lane < 2 * kHalfRowsPerWave && row < row_end && row < lattice_rows) {
    const int b = find_utterance(row_splits, N, row);
    const int U = target_lengths[b];
    const int u = (int)(row - row_splits[b]) % (U + 1 > 0 ? U + 1 : 1);
    int col = blank;
    bool ok = true;
    if (which == 1) {
      ok = u < U && u < targets_cols;
      if (ok) {
        col = targets[(int64_t)b * targets_cols + u];
        ok = (unsigned)col < (unsigned)V;
      }
    }
    lp[2 * row + which] = ok ? to_float<E>(logits[row * (int64_t)V + col]) - d : OT_NEG_INF;
  }
}

// 8 elements of a 16-byte access
template <class E>
__device__ __forceinline__ void unpack8(u32x4 raw, float (&v)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = to_float<E>((unsigned short)(raw[i] & 0xffffu));
    v[2 * i + 1] = to_float<E>((unsigned short)(raw[i] >> 16));
  }
}

// Rows of 2V bytes start at any even byte offset.  For a 16-byte aligned array the
// denominator pass still moves 16 aligned bytes per lane: a group of L lanes reads
// the K * L aligned 16-byte pieces that cover its row, starting at the boundary at
// or below the row's first byte, and elements of the neighbouring rows in the first
// and the last piece are masked.  Ordinary (cached) loads: neighbouring rows share
// those pieces.  The wave's rows are one raw buffer, so the last piece of the last
// row may reach past the array: it reads zeros there, which are masked like the rest.
template <class E, int L, int K>
__global__ __launch_bounds__(kBlock) void lse_gather_half_wide_kernel(
    const unsigned short *__restrict__ logits, const int32_t *__restrict__ targets,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits, int N,
    int targets_cols, int64_t rows, int V, int blank, float *__restrict__ den,
    float *__restrict__ lp) {
  constexpr int G = kWave / L;
  static_assert(kHalfRowsPerWave % G == 0, "rows per pass");
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave_global = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  const int64_t row_first = wave_global * kHalfRowsPerWave;
  if (row_first >= rows) return;
  const int64_t row_end = min(rows, row_first + kHalfRowsPerWave);
  const int sub = lane % L, g = lane / L;
  const unsigned row_bytes = (unsigned)V * 2u;
  const int64_t byte0 = row_first * (int64_t)V * 2;
  const unsigned shift = (unsigned)(byte0 & 15);
  // size rounded up to whole dwords (the bounds check is per dword): with an odd number
  // of elements the last one shares its aligned dword with two bytes past the array
  const __amdgpu_buffer_rsrc_t buf =
      make_buffer(reinterpret_cast<const char *>(logits) + (byte0 - shift),
                  ((unsigned)(row_end - row_first) * row_bytes + shift + 3u) & ~3u);
  float dvec = 0.f;
  for (int r0 = 0; r0 < kHalfRowsPerWave; r0 += G) {
    if (row_first + r0 >= row_end) break;
    // bytes [rs, rs + row_bytes) of the buffer are this group's row (a row past the
    // wave's last one lies past the buffer: every element masked or zero)
    const unsigned rs = shift + (unsigned)(r0 + g) * row_bytes;
    const unsigned a = rs & ~15u;
    float x[K][8];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const unsigned off = a + (unsigned)(k * L + sub) * 16u;
      unpack8<E>(__builtin_amdgcn_raw_buffer_load_b128(buf, off, 0, 0), x[k]);
      const unsigned lo = rs - off;  // byte offset of the row's first element in this piece
      if (off < rs || off + 16u > rs + row_bytes) {  // a piece at either end of the row
#pragma unroll
        for (int e = 0; e < 8; ++e)
          x[k][e] = ((unsigned)(2 * e) - lo < row_bytes) ? x[k][e] : OT_NEG_INF;
      }
    }
    float cm = OT_NEG_INF;
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) cm = fmaxf(cm, x[k][e]);
    float m = group_allreduce<L>(cm, MaxOp());
    if (__builtin_isinf(m)) m = 0.f;  // as ATen's logsumexp does for an all -inf / +inf row
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += exp_fast(x[k][e] - m);
    const float s = group_allreduce<L>(acc, SumOp());
    const float d = logf(s) + m;
    const float t = __shfl(d, ((lane - r0) & (G - 1)) * L, kWave);
    dvec = (lane >= r0 && lane < r0 + G) ? t : dvec;
  }
  finish_rows<E>(dvec, lane, row_first, row_end, logits, targets, target_lengths, row_splits, N,
                 targets_cols, V, blank, den, lp);
}

// V a multiple of 4 and at most 4 * 32 * 8 elements, array 16-byte aligned: the
// layout of the float32 denominator kernel.  A group of L lanes reduces one row (K
// 8-byte vectors per lane), a wave G = 64 / L rows per pass.  The G rows of a pass
// are contiguous, so the wave reads them as one flat span (lane i takes 16-byte units
// i, i + 64, ...: every load instruction covers an aligned, contiguous 1 KiB) and
// re-shapes the span into the row-group layout through a wave-private LDS buffer;
// the span of the next pass is in flight while the current one is reduced.  The
// blank/target gather reads LDS, and the workgroup's results leave in two contiguous
// pieces at the end.
template <class E, int L, int K>
__global__ __launch_bounds__(kBlock) void lse_gather_half_flat_kernel(
    const unsigned short *__restrict__ logits, const int32_t *__restrict__ targets,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits, int N,
    int targets_cols, int64_t rows, int V, int blank, int rows_per_block, float *__restrict__ den,
    float *__restrict__ lp) {
  constexpr int G = kWave / L;
  constexpr int KS = K / 2;  // 16-byte units per lane and span
  static_assert(G >= 2 && K >= 2 && K % 2 == 0, "span of whole 16-byte units");
  constexpr int kStageBytes = kWave * KS * 16;  // = G * L * K 8-byte vectors
  __shared__ BlockUtterances bu;
  __shared__ __attribute__((aligned(16))) unsigned char s_stage[kWavesPerBlock * kStageBytes];
  __shared__ float s_den[kMaxRowsPerBlock], s_lp[2 * kMaxRowsPerBlock];
  const int64_t row_first = (int64_t)blockIdx.x * rows_per_block;
  const int64_t row_end = min(rows, row_first + rows_per_block);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int sub = lane % L, g = lane / L;
  const int nvec = V / 4;
  unsigned char *stage = s_stage + wave * kStageBytes;

  // the workgroup's rows are one raw buffer: the tail of the last span (rows past
  // row_end) reads as zeros without a bounds branch
  const __amdgpu_buffer_rsrc_t block_buf =
      make_buffer(logits + row_first * (int64_t)V, (unsigned)((row_end - row_first) * V * 2));
  u32x4 a[KS];
  auto issue_span = [&](int64_t base) {
    const unsigned off0 = (unsigned)(base - row_first) * (unsigned)V * 2u;
#pragma unroll
    for (int k = 0; k < KS; ++k)
      a[k] = __builtin_amdgcn_raw_buffer_load_b128(block_buf, off0 + (unsigned)(k * kWave + lane) * 16u,
                                                   0, kAuxStream);
  };

  int64_t base = row_first + (int64_t)wave * G;
  if (base < row_end) issue_span(base);
  // the utterance table is only needed for the gather at the end of a pass: its
  // searches run while the first span is in flight
  bu.load(row_splits, N, row_first, row_end - 1);
  const int64_t lattice_rows = row_splits[N];

  for (; base < row_end; base += kWavesPerBlock * G) {
    const int64_t row = base + g;
    const bool active = row < row_end;
#pragma unroll
    for (int k = 0; k < KS; ++k)
      *reinterpret_cast<u32x4 *>(stage + (k * kWave + lane) * 16) = a[k];
    issue_span(base + kWavesPerBlock * G);  // past row_end: all zeros, never used
    float x[K][4];
    float cm = OT_NEG_INF;
    // two elements of -inf in the array's type: slots past the row's end are replaced by
    // them before the conversion (rows past row_end compute values nobody uses)
    constexpr unsigned kNegInfPair = std::is_same<E, BF16>::value ? 0xff80ff80u : 0xfc00fc00u;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int j = k * L + sub;
      // always inside the wave's buffer
      uint2 r = *reinterpret_cast<const uint2 *>(stage + (g * nvec + j) * 8);
      const bool keep = j < nvec;
      r.x = keep ? r.x : kNegInfPair;
      r.y = keep ? r.y : kNegInfPair;
      x[k][0] = to_float<E>((unsigned short)(r.x & 0xffffu));
      x[k][1] = to_float<E>((unsigned short)(r.x >> 16));
      x[k][2] = to_float<E>((unsigned short)(r.y & 0xffffu));
      x[k][3] = to_float<E>((unsigned short)(r.y >> 16));
#pragma unroll
      for (int e = 0; e < 4; ++e) cm = fmaxf(cm, x[k][e]);
    }
    float m = group_allreduce<L>(cm, MaxOp());
    if (__builtin_isinf(m)) m = 0.f;  // as ATen's logsumexp does for an all -inf / +inf row
    // exp(x - m) = 2^(x * log2(e) - m * log2(e)): one fused multiply-add per element.  The
    // rounding of m * log2(e) shifts every term of the row by the same factor, at most
    // half an ulp of m in the logarithm of the sum, i.e. less than one ulp of the result.
    constexpr float kLog2e = 1.44269502162933349609375f;
    const float mshift = -m * kLog2e;
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc += __builtin_amdgcn_exp2f(__builtin_fmaf(x[k][e], kLog2e, mshift));
    const float d = logf(group_allreduce<L>(acc, SumOp())) + m;

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
        float v = 0.f;
        if (ok) v = to_float<E>(reinterpret_cast<const unsigned short *>(stage)[g * V + col]);
        s_lp[2 * local + sub] = ok ? v - d : OT_NEG_INF;
      }
    }
  }
  __syncthreads();
  const int nrows = (int)(row_end - row_first);
  const int nlp = 2 * (int)max((int64_t)0, min((int64_t)nrows, lattice_rows - row_first));
  for (int i = threadIdx.x; i < nrows; i += kBlock) den[row_first + i] = s_den[i];
  for (int i = threadIdx.x; i < nlp; i += kBlock) lp[2 * row_first + i] = s_lp[i];
}

// A group of L lanes reduces one row (L * kHalfK * VEC >= V), so a wave reduces
// 64 / L rows per pass with DPP butterflies; L = 0 stands for rows of any length
// (whole wave per row, running maximum).  The wave first reduces its
// kHalfRowsPerWave rows and keeps row r's denominator in lane r; then lane pair
// (2r, 2r+1) gathers the blank and the target value of row r, so that the
// dependent reads of the gather (row offsets, target, logit) cost one round trip
// per wave instead of one per row.
constexpr int kHalfK = 8;  // accesses per lane and row

template <class E, int VEC, int L>
__global__ __launch_bounds__(kBlock) void lse_gather_half_kernel(
    const unsigned short *__restrict__ logits, const int32_t *__restrict__ targets,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits, int N,
    int targets_cols, int64_t rows, int V, int blank, float *__restrict__ den,
    float *__restrict__ lp) {
  static_assert(2 * kHalfRowsPerWave <= kWave, "rows per wave");
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave_global = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  const int64_t row_first = wave_global * kHalfRowsPerWave;
  if (row_first >= rows) return;
  const int64_t row_end = min(rows, row_first + kHalfRowsPerWave);
  float dvec = 0.f;  // lane r: denominator of row row_first + r
  if (L > 0) {
    constexpr int LL = L > 0 ? L : kWave;
    constexpr int G = kWave / LL;
    static_assert(kHalfRowsPerWave % G == 0, "rows per pass");
    const int sub = lane % LL, g = lane / LL;
#pragma unroll 2
    for (int r0 = 0; r0 < kHalfRowsPerWave; r0 += G) {
      if (row_first + r0 >= row_end) break;
      const unsigned short *p = logits + min(row_first + r0 + g, row_end - 1) * (int64_t)V;
      float x[kHalfK][VEC];
      float cm = OT_NEG_INF;
#pragma unroll
      for (int k = 0; k < kHalfK; ++k) {
        const int j = (k * LL + sub) * VEC;
        if (j < V) {
          HalfIO<E, VEC>::load_cached(p + j, x[k]);
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) x[k][e] = OT_NEG_INF;
        }
      }
#pragma unroll
      for (int k = 0; k < kHalfK; ++k)
#pragma unroll
        for (int e = 0; e < VEC; ++e) cm = fmaxf(cm, x[k][e]);
      float m = group_allreduce<LL>(cm, MaxOp());
      if (__builtin_isinf(m)) m = 0.f;  // as ATen's logsumexp does for an all -inf / +inf row
      float acc = 0.f;
#pragma unroll
      for (int k = 0; k < kHalfK; ++k)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc += exp_fast(x[k][e] - m);
      const float s = group_allreduce<LL>(acc, SumOp());
      const float d = logf(s) + m;
      // lane r0 + i takes the result of group i
      const float t = __shfl(d, ((lane - r0) & (G - 1)) * LL, kWave);
      dvec = (lane >= r0 && lane < r0 + G) ? t : dvec;
    }
  } else {
    constexpr int kChunk = kWave * VEC;
    for (int r = 0; row_first + r < row_end; ++r) {
      const unsigned short *p = logits + (row_first + r) * (int64_t)V;
      float lm = OT_NEG_INF, ls = 0.f;
      for (int j = lane * VEC; j < V; j += kChunk) {
        float x[VEC];
        HalfIO<E, VEC>::load_cached(p + j, x);
        float cm = OT_NEG_INF;
#pragma unroll
        for (int e = 0; e < VEC; ++e) cm = fmaxf(cm, x[e]);
        const float nm = fmaxf(lm, cm);
        const float ref = __builtin_isinf(nm) ? 0.f : nm;
        float acc = (ls == 0.f) ? 0.f : ls * exp_fast((__builtin_isinf(lm) ? 0.f : lm) - ref);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc += exp_fast(x[e] - ref);
        ls = acc;
        lm = nm;
      }
      float m = group_allreduce<kWave>(lm, MaxOp());
      if (__builtin_isinf(m)) m = 0.f;
      const float lref = __builtin_isinf(lm) ? 0.f : lm;
      const float part = (ls == 0.f) ? 0.f : ls * exp_fast(lref - m);
      const float s = group_allreduce<kWave>(part, SumOp());
      const float d = logf(s) + m;
      dvec = (lane == r) ? d : dvec;
    }
  }

  finish_rows<E>(dvec, lane, row_first, row_end, logits, targets, target_lengths, row_splits, N,
                 targets_cols, V, blank, den, lp);
}

// log-softmax input: lp is the two gathered values themselves
template <class E>
__global__ __launch_bounds__(kBlock) void gather_half_kernel(
    const unsigned short *__restrict__ logits, const int32_t *__restrict__ targets,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits, int N,
    int targets_cols, int64_t rows, int V, int blank, float *__restrict__ lp) {
  const int64_t lattice_rows = min(rows, (int64_t)row_splits[N]);
  const int64_t row = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (row >= lattice_rows) return;
  const unsigned short *p = logits + row * (int64_t)V;
  const float bl = to_float<E>(p[blank]);
  const int b = find_utterance(row_splits, N, row);
  const int U = target_lengths[b];
  const int u = (int)(row - row_splits[b]) % (U + 1 > 0 ? U + 1 : 1);
  float sym = OT_NEG_INF;
  if (u < U && u < targets_cols) {
    const int col = targets[(int64_t)b * targets_cols + u];
    if ((unsigned)col < (unsigned)V) sym = to_float<E>(p[col]);
  }
  reinterpret_cast<float2 *>(lp)[row] = make_float2(bl, sym);
}

// ---------------------------------------------------------------------------
// gradient: flat pass over the (rows, V) array, 16 bytes (8 elements) per access
// whatever V is.  S = the largest of 8, 4, 2, 1 that divides V: S consecutive
// elements that start at a multiple of S lie in one row, so an access is
// 8 / S pieces; for V >= 8 they belong to at most two rows (a 2V-byte row need
// not be a multiple of 16 bytes).  The per-row coefficients are those of
// row_coeff_kernel.
// ---------------------------------------------------------------------------
constexpr int kHalfGradUnroll = 2;  // accesses per thread
constexpr int kHalfWide = 8;        // elements per access

// Gradient of S consecutive elements of one row, columns col0 .. col0 + S - 1.
// The result is rounded to 8 or 11 significant bits, so the common entries take
// the one-multiply exponential (relative error 1e-7 + |argument| * 9e-8, below
// 2e-7 absolute for values <= 1); the two special columns, where two terms may
// cancel, keep the accurate one.
template <int S, bool FLS>
__device__ __forceinline__ void grad_piece(const float *x, float *y, const float4 f, const int2 ci,
                                           int col0, float scale, float factor) {
  // the two special columns are rarely among these S: one test for the piece
  const unsigned d1 = (unsigned)(ci.x - col0), d2 = (unsigned)(ci.y - col0);
  const bool special = d1 < (unsigned)S || d2 < (unsigned)S;
  if (FLS) {
#pragma unroll
    for (int e = 0; e < S; ++e) y[e] = 0.f;
    if (special) {
#pragma unroll
      for (int e = 0; e < S; ++e) {
        if (d1 == (unsigned)e) y[e] = f.x * factor;
        if (d2 == (unsigned)e) y[e] = f.y * factor;
      }
    }
  } else {
    // exp(x + shift) = 2^(x * log2(e) + shift * log2(e)): one fused multiply-add and one
    // hardware 2^x per element
    constexpr float kLog2e = 1.44269502162933349609375f;
    const float shift = (f.x + f.y) * kLog2e;
    if (ci.x == kZeroRow) {  // exact zeros whatever the logits hold
#pragma unroll
      for (int e = 0; e < S; ++e) y[e] = 0.f;
      return;
    }
#pragma unroll
    for (int e = 0; e < S; ++e) y[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[e], kLog2e, shift));
    if (special) {
      // at most one element per special column: pick it, evaluate the two accurate
      // exponentials once, and put the difference back
      if (d1 < (unsigned)S) {
        float xe = x[0];
#pragma unroll
        for (int e = 1; e < S; ++e) xe = (d1 == (unsigned)e) ? x[e] : xe;
        const float v = exp_any((xe + f.x) + f.y) - exp_any((xe + f.x) + f.z);
#pragma unroll
        for (int e = 0; e < S; ++e) y[e] = (d1 == (unsigned)e) ? v : y[e];
      }
      if (d2 < (unsigned)S) {
        float xe = x[0];
#pragma unroll
        for (int e = 1; e < S; ++e) xe = (d2 == (unsigned)e) ? x[e] : xe;
        const float v = exp_any((xe + f.x) + f.y) - exp_any((xe + f.x) + f.w);
#pragma unroll
        for (int e = 0; e < S; ++e) y[e] = (d2 == (unsigned)e) ? v : y[e];
      }
    }
    if (scale != 1.f) {
#pragma unroll
      for (int e = 0; e < S; ++e) y[e] *= scale;
    }
  }
}

template <class E>
__device__ __forceinline__ u32x4 pack8(const float (&v)[8]) {
  u32x4 raw;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    raw[i] = (unsigned)from_float<E>(v[2 * i]) | ((unsigned)from_float<E>(v[2 * i + 1]) << 16);
  return raw;
}

// V >= 8.  A workgroup owns kHalfGradUnroll * 256 consecutive 16-byte accesses as one
// raw buffer (the tail of the last workgroup needs no branch); the coefficients of
// the access's first row and of the row after it are both loaded up front, and each
// piece picks one of the two without a branch.
template <class E, int S, bool FLS>
__global__ __launch_bounds__(kBlock) void grad_flat_half_kernel(
    const unsigned short *logits, unsigned short *grad, const float4 *__restrict__ coef_f,
    const int2 *__restrict__ coef_i, int64_t total, int64_t last_row, int V, float inv_v,
    double inv_v_d, float scale, const float *__restrict__ device_factor) {
  const float factor = device_factor ? *device_factor : 1.f;
  if (!FLS) scale *= factor;
  constexpr int kPerBlock = kHalfGradUnroll * kBlock * kHalfWide;  // elements per workgroup
  // Every XCD takes runs of 16 consecutive workgroups' worth of the array (128 KB): the
  // 24-byte row coefficients, which several neighbouring workgroups share, are then fetched
  // into one L2 instead of up to eight (2-byte rows are half as long, so the eightfold
  // fetch weighs twice what it does for float32 logits), +4-6 % for the in-place stream.
  // Runs of 8 help less, 32 and runs that are no power of two not at all; the float32
  // kernel loses 2-6 % with any such mapping.
  const unsigned lblock = xcd_run_block(blockIdx.x, gridDim.x, 16u);
  const int64_t base = (int64_t)lblock * kPerBlock;
  // base / V through a double reciprocal (exact below 2^53) and one correction step
  int64_t row_base = (int64_t)((double)base * inv_v_d);
  {
    const int64_t r = base - row_base * V;
    if (r < 0) --row_base; else if (r >= V) ++row_base;
  }
  const int rem_base = (int)(base - row_base * V);
  const int64_t wide_end = total - total % kHalfWide;  // whole 16-byte accesses end here
  const unsigned span_bytes =
      (unsigned)max((int64_t)0, min((int64_t)kPerBlock, wide_end - base)) * 2u;
  const __amdgpu_buffer_rsrc_t in_buf = make_buffer((FLS ? grad : logits) + base, span_bytes);
  const __amdgpu_buffer_rsrc_t out_buf = make_buffer(grad + base, span_bytes);

  u32x4 raw[kHalfGradUnroll];
  int rows[kHalfGradUnroll], col0[kHalfGradUnroll];
#pragma unroll
  for (int k = 0; k < kHalfGradUnroll; ++k) {
    const int local = (k * kBlock + (int)threadIdx.x) * kHalfWide;
    if (!FLS) raw[k] = __builtin_amdgcn_raw_buffer_load_b128(in_buf, (unsigned)local * 2u, 0, kAuxStream);
    // row and column of the access's first element: idx < V + kPerBlock is exact in
    // float, one correction step fixes the quotient
    const int idx = rem_base + local;
    int q = (int)((float)idx * inv_v);
    if (q * V > idx) --q; else if ((q + 1) * V <= idx) ++q;
    rows[k] = q;
    col0[k] = idx - q * V;
  }
  float4 f0[kHalfGradUnroll], f1[kHalfGradUnroll];
  int2 c0[kHalfGradUnroll], c1[kHalfGradUnroll];
#pragma unroll
  for (int k = 0; k < kHalfGradUnroll; ++k) {
    const int64_t row0 = min(row_base + rows[k], last_row);
    f0[k] = coef_f[row0];
    c0[k] = coef_i[row0];
    if (S < kHalfWide) {
      const int64_t row1 = min(row0 + 1, last_row);
      f1[k] = coef_f[row1];
      c1[k] = coef_i[row1];
    }
  }
#pragma unroll
  for (int k = 0; k < kHalfGradUnroll; ++k) {
    const int local = (k * kBlock + (int)threadIdx.x) * kHalfWide;
    float x[kHalfWide], y[kHalfWide];
    if (!FLS) unpack8<E>(raw[k], x);
#pragma unroll
    for (int j = 0; j < kHalfWide; j += S) {
      const int cj = col0[k] + j;
      const bool second = S < kHalfWide && cj >= V;  // S divides V: a piece never straddles
      const float4 f = second ? f1[k] : f0[k];
      const int2 ci = second ? c1[k] : c0[k];
      grad_piece<S, FLS>(&x[j], &y[j], f, ci, second ? cj - V : cj, scale, factor);
    }
    __builtin_amdgcn_raw_buffer_store_b128(pack8<E>(y), out_buf, (unsigned)local * 2u, 0,
                                           kAuxStreamStore);
  }
  // the last total % 8 elements (a multiple of S), S at a time
  if (S < kHalfWide && lblock == gridDim.x - 1) {
    const int64_t elem = wide_end + (int64_t)threadIdx.x * S;
    if (elem < total) {
      float xs[S], ys[S];
      if (!FLS) HalfIO<E, S>::load(logits + elem, xs);
      const int64_t row = elem / V;
      grad_piece<S, FLS>(xs, ys, coef_f[row], coef_i[row], (int)(elem - row * V), scale, factor);
      HalfIO<E, S>::store(grad + elem, ys);
    }
  }
}

// the same pass with S elements per access, for buffers that are not 16-byte aligned
template <class E, int S, bool FLS>
__global__ __launch_bounds__(kBlock) void grad_flat_half_narrow_kernel(
    const unsigned short *logits, unsigned short *grad, const float4 *__restrict__ coef_f,
    const int2 *__restrict__ coef_i, int64_t nunits, int nvec, float scale,
    const float *__restrict__ device_factor) {
  const float factor = device_factor ? *device_factor : 1.f;
  if (!FLS) scale *= factor;
#pragma unroll
  for (int k = 0; k < kHalfGradUnroll; ++k) {
    const int64_t unit = ((int64_t)blockIdx.x * kHalfGradUnroll + k) * kBlock + threadIdx.x;
    if (unit >= nunits) return;
    const int64_t row = unit / nvec;
    float x[S], y[S];
    if (!FLS) HalfIO<E, S>::load(logits + unit * S, x);
    grad_piece<S, FLS>(x, y, coef_f[row], coef_i[row], (int)(unit - row * nvec) * S, scale, factor);
    HalfIO<E, S>::store(grad + unit * S, y);
  }
}

// x *= *factor for 2-byte elements, skipped on the device when *factor == 1
template <class E>
__global__ __launch_bounds__(kBlock) void scale_half_kernel(unsigned short *__restrict__ x,
                                                            int64_t n,
                                                            const float *__restrict__ factor) {
  const float f = *factor;
  if (f == 1.f) return;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    const int64_t n8 = n / 8;
    for (int64_t i = tid; i < n8; i += stride) {
      float v[8];
      HalfIO<E, 8>::load(x + i * 8, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] *= f;
      HalfIO<E, 8>::store(x + i * 8, v);
    }
    for (int64_t i = n8 * 8 + tid; i < n; i += stride) x[i] = from_float<E>(to_float<E>(x[i]) * f);
  } else {
    for (int64_t i = tid; i < n; i += stride) x[i] = from_float<E>(to_float<E>(x[i]) * f);
  }
}

static inline int launch_status() { return (int)hipGetLastError(); }

static inline int width_for(int V, const void *a, const void *b) {
  const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b);
  int vec = 8;
  while (vec > 1 && (V % vec != 0 || (bits & (uintptr_t)(vec * 2 - 1)) != 0)) vec >>= 1;
  return vec;
}

template <class E>
static int launch_log_probs(const unsigned short *logits, const int32_t *targets,
                            const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                            int32_t targets_cols, int64_t rows, int32_t V, int32_t blank,
                            int32_t from_log_softmax, float *den, float *lp, hipStream_t s) {
  if (from_log_softmax) {
    const unsigned blocks = (unsigned)((rows + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(gather_half_kernel<E>, dim3(blocks), dim3(kBlock), 0, s, logits, targets,
                       target_lengths, row_splits, N, targets_cols, rows, V, blank, lp);
    return launch_status();
  }
  if ((reinterpret_cast<uintptr_t>(logits) & 15) == 0 && V % 4 == 0) {
    // rows as one flat stream, re-shaped through LDS
    const int nvec = V / 4;
    int L = 8;
    while (L < 32 && L * 8 < nvec) L *= 2;
    int K = 2;
    while (K < 8 && L * K < nvec) K *= 2;
    if (L * K >= nvec) {
      // about 256 KiB of logits per workgroup, a whole number of wave passes
      const int pass = kWavesPerBlock * (kWave / L);
      int rpb = (int)((256 * 1024 / ((int64_t)V * 2)) / pass * pass);
      if (rpb < pass) rpb = pass;
      if (rpb > kMaxRowsPerBlock) rpb = kMaxRowsPerBlock;
      const unsigned nblocks = (unsigned)((rows + rpb - 1) / rpb);
#define OT_LAUNCH_LSEF(L_, K_)                                                                    \
  hipLaunchKernelGGL((lse_gather_half_flat_kernel<E, L_, K_>), dim3(nblocks), dim3(kBlock), 0, s, \
                     logits, targets, target_lengths, row_splits, N, targets_cols, rows, V, blank, \
                     rpb, den, lp)
#define OT_LAUNCH_LSEF_K(L_)                 \
  switch (K) {                               \
    case 2: OT_LAUNCH_LSEF(L_, 2); break;    \
    case 4: OT_LAUNCH_LSEF(L_, 4); break;    \
    default: OT_LAUNCH_LSEF(L_, 8); break;   \
  }
      switch (L) {
        case 8: OT_LAUNCH_LSEF_K(8) break;
        case 16: OT_LAUNCH_LSEF_K(16) break;
        default: OT_LAUNCH_LSEF_K(32) break;
      }
#undef OT_LAUNCH_LSEF_K
#undef OT_LAUNCH_LSEF
      return launch_status();
    }
  }
  const int64_t rows_per_block = (int64_t)kWavesPerBlock * kHalfRowsPerWave;
  const unsigned blocks = (unsigned)((rows + rows_per_block - 1) / rows_per_block);
  if ((reinterpret_cast<uintptr_t>(logits) & 15) == 0) {
    // aligned 16-byte pieces that cover a row wherever it starts
    const int pieces = (V * 2) % 16 == 0 ? V / 8 : (V * 2 + 14 + 15) / 16;
    const int K = pieces <= 4 * kWave ? 4 : 8;
    int L = 8;
    while (L < kWave && L * K < pieces) L *= 2;
    if (L * K >= pieces) {
#define OT_LAUNCH_LSEW(L_, K_)                                                                    \
  hipLaunchKernelGGL((lse_gather_half_wide_kernel<E, L_, K_>), dim3(blocks), dim3(kBlock), 0, s,  \
                     logits, targets, target_lengths, row_splits, N, targets_cols, rows, V, blank, \
                     den, lp)
      if (K == 4) {
        switch (L) {
          case 8: OT_LAUNCH_LSEW(8, 4); break;
          case 16: OT_LAUNCH_LSEW(16, 4); break;
          case 32: OT_LAUNCH_LSEW(32, 4); break;
          default: OT_LAUNCH_LSEW(64, 4); break;
        }
      } else {
        OT_LAUNCH_LSEW(64, 8);
      }
#undef OT_LAUNCH_LSEW
      return launch_status();
    }
  }
  const int vec = width_for(V, logits, nullptr);
  // lanes per row: the smallest of 8, 16, 32, 64 with L * kHalfK accesses covering a row
  const int nunits = (V + vec - 1) / vec;
  int L = 8;
  while (L < kWave && L * kHalfK < nunits) L *= 2;
  if (L * kHalfK < nunits) L = 0;
#define OT_LAUNCH_LSEH(VEC_, L_)                                                                  \
  hipLaunchKernelGGL((lse_gather_half_kernel<E, VEC_, L_>), dim3(blocks), dim3(kBlock), 0, s,     \
                     logits, targets, target_lengths, row_splits, N, targets_cols, rows, V, blank, \
                     den, lp)
#define OT_LAUNCH_LSEH_K(VEC_)                                                        \
  switch (L) {                                                                        \
    case 8: OT_LAUNCH_LSEH(VEC_, 8); break;                                           \
    case 16: OT_LAUNCH_LSEH(VEC_, 16); break;                                         \
    case 32: OT_LAUNCH_LSEH(VEC_, 32); break;                                         \
    case 64: OT_LAUNCH_LSEH(VEC_, 64); break;                                         \
    default: OT_LAUNCH_LSEH(VEC_, 0); break;                                          \
  }
  switch (vec) {
    case 8: OT_LAUNCH_LSEH_K(8) break;
    case 4: OT_LAUNCH_LSEH_K(4) break;
    case 2: OT_LAUNCH_LSEH_K(2) break;
    default: OT_LAUNCH_LSEH_K(1) break;
  }
#undef OT_LAUNCH_LSEH_K
#undef OT_LAUNCH_LSEH
  return launch_status();
}

template <class E>
static int launch_gradient(const unsigned short *logits, const void *row_scratch, int64_t rows,
                           int32_t V, int32_t from_log_softmax, float grad_scale,
                           const float *device_factor, unsigned short *grad, hipStream_t s) {
  const float4 *coef_f = static_cast<const float4 *>(row_scratch);
  const int2 *coef_i = reinterpret_cast<const int2 *>(coef_f + rows);
  int S = 8;  // elements that never straddle two rows
  while (S > 1 && V % S != 0) S >>= 1;
  const uintptr_t bits = reinterpret_cast<uintptr_t>(grad) |
                         (from_log_softmax ? 0 : reinterpret_cast<uintptr_t>(logits));
  const int64_t total = rows * (int64_t)V;
  if ((bits & 15) == 0 && V >= kHalfWide && V < (1 << 23)) {
    const int64_t per_block = (int64_t)kHalfGradUnroll * kBlock * kHalfWide;
    const int64_t blocks = (total + per_block - 1) / per_block;
    if (blocks > INT32_MAX) return OT_E_BAD_ARG;
#define OT_LAUNCH_GRADH(S_, FLS_)                                                               \
  hipLaunchKernelGGL((grad_flat_half_kernel<E, S_, FLS_>), dim3((unsigned)blocks), dim3(kBlock), \
                     0, s, logits, grad, coef_f, coef_i, total, rows - 1, V, 1.0f / (float)V,   \
                     1.0 / (double)V, grad_scale, device_factor)
#define OT_LAUNCH_GRADH_S(FLS_)                        \
  switch (S) {                                         \
    case 8: OT_LAUNCH_GRADH(8, FLS_); break;           \
    case 4: OT_LAUNCH_GRADH(4, FLS_); break;           \
    case 2: OT_LAUNCH_GRADH(2, FLS_); break;           \
    default: OT_LAUNCH_GRADH(1, FLS_); break;          \
  }
    if (from_log_softmax) { OT_LAUNCH_GRADH_S(true) } else { OT_LAUNCH_GRADH_S(false) }
#undef OT_LAUNCH_GRADH_S
#undef OT_LAUNCH_GRADH
    return launch_status();
  }
  // narrow accesses: S limited by the alignment of the buffers as well
  while (S > 1 && (bits & (uintptr_t)(S * 2 - 1)) != 0) S >>= 1;
  const int nvec = V / S;
  const int64_t nunits = rows * nvec;
  const int64_t per_block = (int64_t)kHalfGradUnroll * kBlock;
  const int64_t blocks = (nunits + per_block - 1) / per_block;
  if (blocks > INT32_MAX) return OT_E_BAD_ARG;
#define OT_LAUNCH_GRADN(S_, FLS_)                                                                \
  hipLaunchKernelGGL((grad_flat_half_narrow_kernel<E, S_, FLS_>), dim3((unsigned)blocks),         \
                     dim3(kBlock), 0, s, logits, grad, coef_f, coef_i, nunits, nvec, grad_scale,  \
                     device_factor)
#define OT_LAUNCH_GRADN_S(FLS_)                        \
  switch (S) {                                         \
    case 8: OT_LAUNCH_GRADN(8, FLS_); break;           \
    case 4: OT_LAUNCH_GRADN(4, FLS_); break;           \
    case 2: OT_LAUNCH_GRADN(2, FLS_); break;           \
    default: OT_LAUNCH_GRADN(1, FLS_); break;          \
  }
  if (from_log_softmax) { OT_LAUNCH_GRADN_S(true) } else { OT_LAUNCH_GRADN_S(false) }
#undef OT_LAUNCH_GRADN_S
#undef OT_LAUNCH_GRADN
  return launch_status();
}

}  // namespace ot

using namespace ot;

extern "C" {

int ot_log_probs_half(const void *logits, int32_t dtype, const int32_t *targets,
                      const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                      int32_t targets_cols, int64_t rows, int32_t V, int32_t blank,
                      int32_t from_log_softmax, float *den, float *lp, void *stream) {
  if (!logits || !lp || !target_lengths || !row_splits || N <= 0 || rows <= 0 ||
      rows > INT32_MAX || V <= 0 || blank < 0 || blank >= V || targets_cols < 0 ||
      (targets_cols > 0 && !targets) || (!from_log_softmax && !den) ||
      (dtype != OT_DTYPE_F16 && dtype != OT_DTYPE_BF16))
    return OT_E_BAD_ARG;
  if (reinterpret_cast<uintptr_t>(logits) & 1) return OT_E_MISALIGNED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned short *p = static_cast<const unsigned short *>(logits);
  return dtype == OT_DTYPE_F16
             ? launch_log_probs<F16>(p, targets, target_lengths, row_splits, N, targets_cols, rows,
                                     V, blank, from_log_softmax, den, lp, s)
             : launch_log_probs<BF16>(p, targets, target_lengths, row_splits, N, targets_cols, rows,
                                      V, blank, from_log_softmax, den, lp, s);
}

int ot_gradient_apply_half(const void *logits, int32_t dtype, const void *row_scratch,
                           int64_t rows, int32_t V, int32_t from_log_softmax, float grad_scale,
                           const float *device_factor, void *grad, void *stream) {
  if (!row_scratch || !grad || rows <= 0 || rows > INT32_MAX || V <= 0 ||
      (dtype != OT_DTYPE_F16 && dtype != OT_DTYPE_BF16))
    return OT_E_BAD_ARG;
  if (from_log_softmax ? grad == logits : !logits) return OT_E_BAD_ARG;
  if ((reinterpret_cast<uintptr_t>(grad) & 1) || (reinterpret_cast<uintptr_t>(logits) & 1) ||
      (reinterpret_cast<uintptr_t>(row_scratch) & 15))
    return OT_E_MISALIGNED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned short *p = static_cast<const unsigned short *>(logits);
  unsigned short *g = static_cast<unsigned short *>(grad);
  return dtype == OT_DTYPE_F16
             ? launch_gradient<F16>(p, row_scratch, rows, V, from_log_softmax, grad_scale,
                                    device_factor, g, s)
             : launch_gradient<BF16>(p, row_scratch, rows, V, from_log_softmax, grad_scale,
                                     device_factor, g, s);
}

int ot_scale_by_device_scalar_half(void *x, int32_t dtype, int64_t n, const float *factor,
                                   void *stream) {
  if (!x || !factor || n < 0 || (dtype != OT_DTYPE_F16 && dtype != OT_DTYPE_BF16))
    return OT_E_BAD_ARG;
  if (reinterpret_cast<uintptr_t>(x) & 1) return OT_E_MISALIGNED;
  if (n == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // 1024 persistent workgroups of 4 KB per sweep (4 MB per sweep of the grid, like the
  // float32 kernel's 256 x 16 KB): 5.8 / 5.3 TB/s on 0.75 / 1.95 GB against 5.3 / 4.7 with
  // 4096 workgroups and 5.2 / 5.0 with 512
  int64_t blocks = (n / 8 + kBlock - 1) / kBlock;
  if (blocks > 1024) blocks = 1024;
  if (blocks < 1) blocks = 1;
  unsigned short *p = static_cast<unsigned short *>(x);
  if (dtype == OT_DTYPE_F16)
    hipLaunchKernelGGL(scale_half_kernel<F16>, dim3((unsigned)blocks), dim3(kBlock), 0, s, p, n, factor);
  else
    hipLaunchKernelGGL(scale_half_kernel<BF16>, dim3((unsigned)blocks), dim3(kBlock), 0, s, p, n, factor);
  return launch_status();
}

}  // extern "C"
