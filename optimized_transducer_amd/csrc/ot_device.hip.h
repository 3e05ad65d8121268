// Device-side building blocks shared by the transducer-loss kernels (gfx950).
//
// Everything here is wave64 code: cross-lane traffic uses DPP controls of the
// GFX9 family (quad_perm, row_mirror, wave_shr/wave_shl) and falls back to the
// LDS crossbar (ds_bpermute via __shfl_xor) only for the two widest butterfly
// steps.
#ifndef OT_DEVICE_HIP_H_
#define OT_DEVICE_HIP_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ot {

constexpr int kWave = 64;
constexpr int kBlock = 256;           // streaming kernels: 4 waves per workgroup
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kMaxRowsPerBlock = 256; // bounds the utterance table kept in LDS

#define OT_NEG_INF (-__builtin_huge_valf())

// logf(FLT_EPSILON): below this difference the smaller term of a two-term
// log-add is dropped (reference optimized_transducer/csrc/cpu.cc:15-16,30-34).
constexpr float kMinLogDiff = -15.9423847198486328125f;

// DPP control words (GFX9 encoding).
constexpr int kDppQuadXor1 = 0xB1;       // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;       // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141; // lane i <-> 7-i inside 8 lanes
constexpr int kDppRowMirror = 0x140;     // lane i <-> 15-i inside 16 lanes
constexpr int kDppWaveShl1 = 0x130;      // lane i reads lane i+1
constexpr int kDppWaveShr1 = 0x138;      // lane i reads lane i-1

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}

// Lane i receives x of lane i-1; lane 0 (which has no source) receives fill.
__device__ __forceinline__ float wave_shift_up(float x, float fill) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, fill),
                                         __builtin_bit_cast(int, x), kDppWaveShr1,
                                         0xf, 0xf, false));
}

// Lane i receives x of lane i+1; lane 63 receives fill.
__device__ __forceinline__ float wave_shift_down(float x, float fill) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, fill),
                                         __builtin_bit_cast(int, x), kDppWaveShl1,
                                         0xf, 0xf, false));
}

struct MaxOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};
struct SumOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};

// All-reduce over aligned groups of L consecutive lanes (L = 1..64, power of
// two).  Butterfly: after step s every lane holds the reduction of its aligned
// 2^s group, so all lanes of a group end with the same bits.
template <int L, class Op>
__device__ __forceinline__ float group_allreduce(float v, Op op) {
  if (L >= 2) v = op(v, dpp_mov<kDppQuadXor1>(v));
  if (L >= 4) v = op(v, dpp_mov<kDppQuadXor2>(v));
  if (L >= 8) v = op(v, dpp_mov<kDppRowHalfMirror>(v));
  if (L >= 16) v = op(v, dpp_mov<kDppRowMirror>(v));
  if (L >= 32) v = op(v, __shfl_xor(v, 16, kWave));
  if (L >= 64) v = op(v, __shfl_xor(v, 32, kWave));
  return v;
}

// exp(x) through the hardware 2^x unit, argument scaled by a rounded log2(e):
// relative error about 1 ulp + |x| * 2^-24.  Used where thousands of terms are
// summed (the softmax denominator), so single-term errors average out.
__device__ __forceinline__ float exp_fast(float x) {
  return __builtin_amdgcn_exp2f(x * 1.44269502162933349609375f);
}

// exp(x) for any x through the hardware 2^x unit, accurate to about 1 ulp:
// the product x*log2(e) is formed in two pieces (rounded product + its exact
// residual) so that the argument error does not grow with |x|.  The limits
// (0, +inf) are passed through, so x = -inf (a masked logit) gives exactly 0.
// Used for the gradient entries.
__device__ __forceinline__ float exp_any(float x) {
  constexpr float kLog2eHi = 1.44269502162933349609375f;  // float(log2(e))
  constexpr float kLog2eLo = 1.92596299112661746e-8f;     // log2(e) - kLog2eHi
  constexpr float kLn2 = 0.693147182464599609375f;
  const float ph = x * kLog2eHi;
  const float pl = __builtin_fmaf(x, kLog2eHi, -ph) + x * kLog2eLo;
  const float e = __builtin_amdgcn_exp2f(ph);
  const float r = __builtin_fmaf(e, pl * kLn2, e);
  return (e == 0.0f || __builtin_isinf(e)) ? e : r;
}

// log(exp(a) + exp(b)) ordered as the reference's CPU LogSumExp (cpu.cc:18-35):
// larger + log1p(exp(smaller - larger)), or just the larger one when the
// difference is below kMinLogDiff or is NaN (-inf minus -inf).  Both
// transcendental steps run straight on the hardware units (2^x and log2);
// absolute error of the added term about 1.5e-7, i.e. below one ulp of the
// result as soon as |larger| >= 2.  This function is the critical path of the
// lattice sweep.
__device__ __forceinline__ float log_add(float a, float b) {
  constexpr float kLog2e = 1.44269502162933349609375f;
  constexpr float kLn2 = 0.693147182464599609375f;
  // smaller - larger = -|a - b| (the sign and abs fold into operand modifiers);
  // (-inf, -inf) still gives a NaN difference, which fails the threshold test
  // below like in the reference
  const float hi = __builtin_fmaxf(a, b);
  const float diff = -__builtin_fabsf(a - b);
  const float e = __builtin_amdgcn_exp2f(diff * kLog2e);
  const float l = __builtin_amdgcn_logf(1.0f + e) * kLn2;
  return hi + ((diff >= kMinLogDiff) ? l : 0.0f);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits
// for every outstanding global load and store of the wave, which would drain
// the lattice sweep's prefetch ring at each barrier; here only the LDS counter
// (lgkmcnt) is waited for.  simm16 0xC07F = vmcnt 63, expcnt 7, lgkmcnt 0.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Raw buffer view of a device array: loads beyond `bytes` return 0 and stores
// beyond it are dropped by the hardware, which removes every bounds branch
// from the lattice sweep.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}

// Largest b in [0, n-1] with splits[b] <= row (splits ascending, splits[0]=0).
__device__ __forceinline__ int find_utterance(const int32_t *splits, int n, int64_t row) {
  int lo = 0, hi = n;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if ((int64_t)splits[mid] <= row) lo = mid; else hi = mid;
  }
  return lo;
}

// find_utterance by a whole wave: every lane returns the number of b in [1, n-1] with
// splits[b] <= row, which is that b (splits ascending, splits[0] = 0 <= row).
__device__ __forceinline__ int find_utterance_wave(const int32_t *__restrict__ splits, int n,
                                                   int64_t row) {
  const int lane = threadIdx.x & (kWave - 1);
  int count = 0;
  for (int base = 1; base < n; base += kWave) {
    const int i = base + lane;
    const bool le = i < n && (int64_t)splits[i] <= row;
    count += __builtin_popcountll(__ballot(le));
  }
  return count;
}

// The wave-parallel count reads the whole table (n/64 rounds of independent loads), the
// binary search log2(n) dependent ones: the first is faster for the few hundred
// utterances of a usual batch, the second for thousands.
constexpr int kWaveSearchMax = 1024;
__device__ __forceinline__ int find_utterance_uniform(const int32_t *__restrict__ splits, int n,
                                                      int64_t row) {
  return n <= kWaveSearchMax ? find_utterance_wave(splits, n, row) : find_utterance(splits, n, row);
}

// Utterance table of one workgroup of a per-row streaming kernel.  A workgroup
// owns a contiguous span of at most kMaxRowsPerBlock rows, which can touch at
// most that many + 1 utterances (every utterance has at least one row), so the
// slice of row_splits it needs always fits this fixed LDS footprint.
struct BlockUtterances {
  int32_t splits[kMaxRowsPerBlock + 2];
  int32_t b_lo, b_hi;  // utterances of the block's first and last row
  // utterances touched
  __device__ __forceinline__ int count() const { return min(b_hi - b_lo + 1, kMaxRowsPerBlock + 1); }

  // Collective over the workgroup (at least one whole wave); row_first <= row_last are
  // the block's rows.  The two searches run in two waves at once (in wave 0 one after
  // the other for a one-wave workgroup), each as one round of 64 parallel comparisons per
  // 64 utterances instead of a chain of log2(N) dependent loads (up to kWaveSearchMax
  // utterances; a binary search beyond).
  __device__ __forceinline__ void load(const int32_t *__restrict__ row_splits, int N,
                                       int64_t row_first, int64_t row_last) {
    const int wave = threadIdx.x / kWave;
    const bool two = blockDim.x >= 2 * kWave;
    if (wave == 0) {
      const int lo = find_utterance_uniform(row_splits, N, row_first);
      if (threadIdx.x == 0) b_lo = lo;
      if (!two) {
        const int hi = find_utterance_uniform(row_splits, N, row_last);
        if (threadIdx.x == 0) b_hi = hi;
      }
    } else if (wave == 1) {
      const int hi = find_utterance_uniform(row_splits, N, row_last);
      if (threadIdx.x == kWave) b_hi = hi;
    }
    __syncthreads();
    const int n = count() + 1;
    for (int i = threadIdx.x; i < n && i < kMaxRowsPerBlock + 2; i += blockDim.x)
      splits[i] = row_splits[b_lo + i];
    __syncthreads();
  }

  // Utterance of a row inside the block's span.
  __device__ __forceinline__ int utterance_of(int64_t row) const {
    return b_lo + find_utterance(splits, count(), row);
  }
  __device__ __forceinline__ int32_t split(int b) const { return splits[b - b_lo]; }
};

// Where a packed row sits in its utterance's lattice.
struct Cell {
  int b, t, u, T, U;
  int64_t row0;  // first row of the utterance
};

__device__ __forceinline__ Cell decode_row(const BlockUtterances &bu, int64_t row,
                                           const int32_t *__restrict__ logit_lengths,
                                           const int32_t *__restrict__ target_lengths) {
  Cell c;
  c.b = bu.utterance_of(row);
  c.row0 = bu.split(c.b);
  c.U = target_lengths[c.b];
  c.T = logit_lengths ? logit_lengths[c.b] : 0;
  const int u1 = c.U + 1 > 0 ? c.U + 1 : 1;
  const int idx = (int)(row - c.row0);
  c.t = idx / u1;
  c.u = idx - c.t * u1;
  return c;
}

// Workgroups are handed to the chip's 8 XCDs (each with its own L2) in turn: workgroup i
// runs on XCD i % 8.  This maps workgroup i to the logical block it should work on such
// that every XCD takes runs of `run` consecutive logical blocks (inside groups of 8 * run
// blocks; the last, partial group keeps the identity), so that small per-row data shared by
// neighbouring blocks is fetched into one L2 instead of several.
__device__ __forceinline__ unsigned xcd_run_block(unsigned bid, unsigned nblocks, unsigned run) {
  const unsigned group = 8u * run;
  const unsigned g = bid / group;
  if (run <= 1u || (g + 1u) * group > nblocks) return bid;
  const unsigned r = bid - g * group;
  return g * group + (r & 7u) * run + (r >> 3);
}

// first column index of a row's gradient coefficients that marks an all-zero row
constexpr int kZeroRow = -2;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
// cache-policy operand of the raw buffer builtins: bit 1 = non-temporal
constexpr int kAuxStream = 2;
// streaming stores: non-temporal plus both scope bits (sc0 sc1, written through);
// 2-4 % faster than non-temporal alone for the in-place and the write-only stream
constexpr int kAuxStreamStore = 19;

// VEC floats of a row.  The (rows, V) arrays are streamed once per kernel and
// never re-read by the same kernel, so their loads and stores carry the
// non-temporal hint (measured on MI355X: ~7.0 vs ~6.3 TB/s for a pure read).
template <int VEC> struct Vec;
template <> struct Vec<4> {
  float v[4];
  __device__ __forceinline__ void load(const float *p) {
    const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
  __device__ __forceinline__ void store(float *p) const {
    const f32x4 x = {v[0], v[1], v[2], v[3]};
    *reinterpret_cast<f32x4 *>(p) = x;
  }
  // ordinary load, for data that is re-read from cache
  __device__ __forceinline__ void load_cached(const float *p) {
    const f32x4 x = *reinterpret_cast<const f32x4 *>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
  __device__ __forceinline__ void load_lds(const float *p) {
    const f32x4 x = *reinterpret_cast<const f32x4 *>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
  // streaming (non-temporal) buffer access: out-of-range reads give 0, writes vanish
  __device__ __forceinline__ void load_buffer(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
    const f32x4 x = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, kAuxStream));
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
  __device__ __forceinline__ void store_buffer(__amdgpu_buffer_rsrc_t r, unsigned byte_off) const {
    const f32x4 x = {v[0], v[1], v[2], v[3]};
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, x), r, byte_off, 0, kAuxStreamStore);
  }
  __device__ __forceinline__ void store_lds(float *p) const { store(p); }
  // for flat, line-aligned streams only: a non-temporal store of a partial
  // cache line is much slower than a cached one
  __device__ __forceinline__ void store_stream(float *p) const {
    const f32x4 x = {v[0], v[1], v[2], v[3]};
    __builtin_nontemporal_store(x, reinterpret_cast<f32x4 *>(p));
  }
};
template <> struct Vec<1> {
  float v[1];
  __device__ __forceinline__ void load(const float *p) { v[0] = __builtin_nontemporal_load(p); }
  __device__ __forceinline__ void store(float *p) const { *p = v[0]; }
  __device__ __forceinline__ void store_stream(float *p) const { __builtin_nontemporal_store(v[0], p); }
  __device__ __forceinline__ void load_lds(const float *p) { v[0] = *p; }
  __device__ __forceinline__ void load_cached(const float *p) { v[0] = *p; }
  __device__ __forceinline__ void load_buffer(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
    v[0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_off, 0, kAuxStream));
  }
  __device__ __forceinline__ void store_buffer(__amdgpu_buffer_rsrc_t r, unsigned byte_off) const {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v[0]), r, byte_off, 0, kAuxStreamStore);
  }
  __device__ __forceinline__ void store_lds(float *p) const { *p = v[0]; }
};

// element types of 2-byte arrays, and their conversions
struct F16 {};   // IEEE binary16
struct BF16 {};  // bfloat16: the upper half of a float32

template <class E> __device__ __forceinline__ float to_float(unsigned short bits);
template <> __device__ __forceinline__ float to_float<F16>(unsigned short bits) {
  return (float)__builtin_bit_cast(_Float16, bits);
}
template <> __device__ __forceinline__ float to_float<BF16>(unsigned short bits) {
  return __builtin_bit_cast(float, (unsigned)bits << 16);
}
template <class E> __device__ __forceinline__ unsigned short from_float(float x);
template <> __device__ __forceinline__ unsigned short from_float<F16>(float x) {
  return __builtin_bit_cast(unsigned short, (_Float16)x);  // round to nearest even
}
template <> __device__ __forceinline__ unsigned short from_float<BF16>(float x) {
  return __builtin_bit_cast(unsigned short, (__bf16)x);  // round to nearest even
}

// element i of an array of float (T = float) or of a 2-byte type (T = F16 / BF16)
template <class T> __device__ __forceinline__ float load_element(const void *p, int64_t i) {
  return to_float<T>(static_cast<const unsigned short *>(p)[i]);
}
template <> __device__ __forceinline__ float load_element<float>(const void *p, int64_t i) {
  return static_cast<const float *>(p)[i];
}

// Gather step alone (ComputeLogProbsForLogSoftmax, kernels.cu:62-88; with `den`,
// ComputeLogProbs, kernels.cu:30-60, for denominators that are already known):
// lp[row] = (logits[row, blank], logits[row, target(row)]) - (den ? den[row] : 0).
// Latency-bound (two dependent small reads per row): a thread works on kGatherRows
// rows at once, starts the reads that need no decoding first and finds its
// utterances with its own binary searches (row_splits stays in L1), so that nothing
// in the workgroup waits for anything else.
constexpr int kGatherRows = 2;

template <class T>
__global__ __launch_bounds__(kBlock) void gather_rows_kernel(
    const void *__restrict__ logits, const float *__restrict__ den,
    const int32_t *__restrict__ targets, const int32_t *__restrict__ target_lengths,
    const int32_t *__restrict__ row_splits, int N, int targets_cols, int64_t row_begin,
    int64_t rows, int V, int blank, float *__restrict__ lp) {
  const int64_t lattice_rows = min(rows, (int64_t)row_splits[N]);
  int64_t row[kGatherRows];
  float bl[kGatherRows], d[kGatherRows];
  int lo[kGatherRows], hi[kGatherRows];
#pragma unroll
  for (int k = 0; k < kGatherRows; ++k) {
    row[k] = row_begin + ((int64_t)blockIdx.x * kGatherRows + k) * kBlock + threadIdx.x;
    const bool in = row[k] < lattice_rows;
    bl[k] = in ? load_element<T>(logits, row[k] * (int64_t)V + blank) : 0.f;
    d[k] = (in && den) ? den[row[k]] : 0.f;
    lo[k] = 0;
    hi[k] = N;
  }
  // largest b with row_splits[b] <= row, all searches in step
  for (int width = N; width > 1; width = (width + 1) >> 1) {
#pragma unroll
    for (int k = 0; k < kGatherRows; ++k) {
      if (hi[k] - lo[k] > 1) {
        const int mid = (lo[k] + hi[k]) >> 1;
        if ((int64_t)row_splits[mid] <= row[k]) lo[k] = mid; else hi[k] = mid;
      }
    }
  }
  int col[kGatherRows];
#pragma unroll
  for (int k = 0; k < kGatherRows; ++k) {
    col[k] = -1;
    if (row[k] < lattice_rows) {
      const int b = lo[k];
      const int U = target_lengths[b];
      const int u1 = U + 1 > 0 ? U + 1 : 1;
      const int u = (int)(row[k] - row_splits[b]) % u1;
      if (u < U && u < targets_cols) col[k] = targets[(int64_t)b * targets_cols + u];
    }
  }
#pragma unroll
  for (int k = 0; k < kGatherRows; ++k) {
    if (row[k] < lattice_rows) {
      float sym = OT_NEG_INF;
      if ((unsigned)col[k] < (unsigned)V)
        sym = load_element<T>(logits, row[k] * (int64_t)V + col[k]) - d[k];
      reinterpret_cast<float2 *>(lp)[row[k]] = make_float2(bl[k] - d[k], sym);
    }
  }
}

}  // namespace ot
#endif  // OT_DEVICE_HIP_H_
