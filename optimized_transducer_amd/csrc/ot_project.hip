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
// Shape of the computation.  A workgroup of 4 waves owns 256 packed rows, a wave 64
// of them, and walks over the vocabulary in passes of 128 columns; per pass a wave
// holds a 128 x 64 block of logits^T in 8 accumulator tiles of 32 x 32
// (v_mfma_f32_32x32x16).  The product is formed transposed (vocabulary along the
// tile's rows, packed rows along its columns) because an accumulator lane then
// holds 16 values of ONE packed row per tile: the running (max, sum) of the row
// stays in that lane and its partner 32 lanes up, with no cross-lane reduction
// until the very end.  W streams through LDS in stages of 32 k-values (shared by the
// 4 waves, double-buffered, 16-byte slots XOR-swizzled against bank conflicts); the
// activations go from global memory straight into the operand registers, 32
// contiguous bytes per lane and stage.  The bias initialises the accumulators.
// Before the store, v_permlane32_swap exchanges half of each tile between a lane
// and its partner so that every lane owns 16 consecutive columns of its row.
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

constexpr int kProjRows = 256;  // packed rows per workgroup
constexpr int kProjCols = 128;  // vocabulary columns per pass
constexpr int kProjK = 32;      // k-values per LDS stage
constexpr int kProjStageBytes = kProjCols * kProjK * 2;

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

// E: element type of x and W.  OUT_F32: logits are float32, else of type E.
// SV: elements per store (SV * element size divides the row pitch and the base).
template <class E, bool OUT_F32, int SV>
__global__ __launch_bounds__(256, 2) void joiner_project_kernel(
    const unsigned short *__restrict__ x, const unsigned short *__restrict__ w,
    const float *__restrict__ bias, int64_t rows, int D, int V, void *__restrict__ logits,
    float *__restrict__ den) {
  __shared__ __attribute__((aligned(16))) unsigned char s_w[2 * kProjStageBytes];
  constexpr unsigned kOutBytes = OUT_F32 ? 4u : 2u;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, h = lane >> 5;
  const int64_t row0 = (int64_t)blockIdx.x * kProjRows;
  const unsigned nrows = (unsigned)min((int64_t)kProjRows, rows - row0);
  // the workgroup's rows, the weight and the bias as raw buffers: rows past the
  // array and vocabulary entries past V read as zeros, stores to them vanish
  const __amdgpu_buffer_rsrc_t xbuf = make_buffer(x + row0 * D, nrows * (unsigned)D * 2u);
  const __amdgpu_buffer_rsrc_t wbuf = make_buffer(w, (unsigned)V * (unsigned)D * 2u);
  const __amdgpu_buffer_rsrc_t bbuf = make_buffer(bias ? bias : den, bias ? (unsigned)V * 4u : 0u);
  const __amdgpu_buffer_rsrc_t obuf =
      make_buffer(static_cast<char *>(logits) + row0 * V * kOutBytes, nrows * (unsigned)V * kOutBytes);

  // operand addressing.  MFMA step ks of a stage: lane group h supplies k-values
  // k0 + 16 h + 8 ks .. + 7 of both operands.
  unsigned xoff[2];
#pragma unroll
  for (int rs = 0; rs < 2; ++rs)
    xoff[rs] = ((unsigned)(64 * wave + 32 * rs + c) * (unsigned)D + 16u * h) * 2u;
  // W stage copy: thread t moves 16-byte pieces p = t, t + 256; piece p is k-chunk p % 4
  // of vocabulary row p / 4 and goes to slot 4 v + (chunk ^ ((v >> 1) & 3))
  unsigned wsrc[2], wdst[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int p = tid + 256 * q, v = p >> 2, cc = p & 3;
    wsrc[q] = ((unsigned)v * (unsigned)D + 8u * cc) * 2u;
    wdst[q] = (unsigned)(4 * v + (cc ^ ((v >> 1) & 3))) * 16u;
  }
  // fragment of vocabulary tile vt, step ks: row 32 vt + c, chunk 2 h + ks
  unsigned wfrag[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) wfrag[ks] = (unsigned)(4 * c + ((2 * h + ks) ^ ((c >> 1) & 3))) * 16u;

  const int ksteps = D / kProjK;
  const int ntiles = (V + kProjCols - 1) / kProjCols;
  const int nstages = ntiles * ksteps;

  u32x4 wreg[2], xreg[2][2], xnext[2][2];
  auto load_stage = [&](int nt, int kk, u32x4 (&xr)[2][2]) {
    const unsigned wbase = ((unsigned)(nt * kProjCols) * (unsigned)D + (unsigned)(kk * kProjK)) * 2u;
#pragma unroll
    for (int q = 0; q < 2; ++q) wreg[q] = __builtin_amdgcn_raw_buffer_load_b128(wbuf, wbase + wsrc[q], 0, 0);
#pragma unroll
    for (int rs = 0; rs < 2; ++rs)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
        xr[rs][ks] = __builtin_amdgcn_raw_buffer_load_b128(
            xbuf, xoff[rs] + (unsigned)(kk * kProjK) * 2u + 16u * ks, 0, 0);
  };
  auto store_stage = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 2; ++q)
      *reinterpret_cast<u32x4 *>(s_w + buf * kProjStageBytes + wdst[q]) = wreg[q];
  };

  float m_run[2] = {OT_NEG_INF, OT_NEG_INF}, s_run[2] = {0.f, 0.f};
  load_stage(0, 0, xreg);
  store_stage(0);
  int stage = 0;
  for (int nt = 0; nt < ntiles; ++nt) {
    const int n0 = nt * kProjCols;
    // accumulators start from the bias: tile (rs, vt), register 4 j + i holds vocabulary
    // entry n0 + 32 vt + 8 j + 4 h + i of packed row 32 rs + c
    f32x16 acc[2][4];
#pragma unroll
    for (int vt = 0; vt < 4; ++vt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 b4 = __builtin_bit_cast(
            f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                       bbuf, (unsigned)(n0 + 32 * vt + 8 * j + 4 * h) * 4u, 0, 0));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[0][vt][4 * j + i] = b4[i];
          acc[1][vt][4 * j + i] = b4[i];
        }
      }
    for (int kk = 0; kk < ksteps; ++kk, ++stage) {
      const bool more = stage + 1 < nstages;
      if (more) {
        const bool wrap = kk + 1 == ksteps;
        load_stage(wrap ? nt + 1 : nt, wrap ? 0 : kk + 1, xnext);
      }
      lds_barrier();  // this stage's W is in LDS; the other buffer is free again
      const unsigned char *sw = s_w + (stage & 1) * kProjStageBytes;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        u32x4 wf[4];
#pragma unroll
        for (int vt = 0; vt < 4; ++vt)
          wf[vt] = *reinterpret_cast<const u32x4 *>(sw + vt * (32 * 4 * 16) + wfrag[ks]);
#pragma unroll
        for (int vt = 0; vt < 4; ++vt)
#pragma unroll
          for (int rs = 0; rs < 2; ++rs)
            acc[rs][vt] = mfma_32x32x16<E>(wf[vt], xreg[rs][ks], acc[rs][vt]);
      }
      if (more) {
        store_stage((stage + 1) & 1);
#pragma unroll
        for (int rs = 0; rs < 2; ++rs)
#pragma unroll
          for (int ks = 0; ks < 2; ++ks) xreg[rs][ks] = xnext[rs][ks];
      }
    }

    // epilogue of the pass: round, update the row's running (max, sum), store
    const bool ragged = n0 + kProjCols > V;  // the last pass may reach past V
#pragma unroll
    for (int rs = 0; rs < 2; ++rs) {
      const unsigned orow = (unsigned)(64 * wave + 32 * rs + c) * (unsigned)V;
#pragma unroll
      for (int vt = 0; vt < 4; ++vt) {
        // after the exchange this lane owns columns vs .. vs + 15 of its row
        const int vs = n0 + 32 * vt + 16 * h;
        float y[16];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const u32x2 r1 = __builtin_amdgcn_permlane32_swap(
              as_u32(acc[rs][vt][i]), as_u32(acc[rs][vt][8 + i]), false, false);
          const u32x2 r2 = __builtin_amdgcn_permlane32_swap(
              as_u32(acc[rs][vt][4 + i]), as_u32(acc[rs][vt][12 + i]), false, false);
          y[i] = as_f32(r1.x);
          y[4 + i] = as_f32(r1.y);
          y[8 + i] = as_f32(r2.x);
          y[12 + i] = as_f32(r2.y);
        }
        unsigned packed[8];
        if (!OUT_F32) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const unsigned short lo = from_float<E>(y[2 * e]), hi = from_float<E>(y[2 * e + 1]);
            packed[e] = (unsigned)lo | ((unsigned)hi << 16);
            y[2 * e] = to_float<E>(lo);
            y[2 * e + 1] = to_float<E>(hi);
          }
        }
        // store: pieces of SV elements; V is a multiple of SV, so a piece is inside the
        // row or past it as a whole
#pragma unroll
        for (int p = 0; p < 16; p += SV) {
          if (vs + p < V) {
            const unsigned off = (orow + (unsigned)(vs + p)) * kOutBytes;
            if (OUT_F32) {
              if (SV == 4) {
                const f32x4 t = {y[p], y[p + 1], y[p + 2], y[p + 3]};
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, t), obuf, off, 0, 0);
              } else if (SV == 2) {
                const u32x2 t = {as_u32(y[p]), as_u32(y[p + 1])};
                __builtin_amdgcn_raw_buffer_store_b64(t, obuf, off, 0, 0);
              } else {
                __builtin_amdgcn_raw_buffer_store_b32(as_u32(y[p]), obuf, off, 0, 0);
              }
            } else {
              if (SV == 8) {
                const u32x4 t = {packed[p / 2], packed[p / 2 + 1], packed[p / 2 + 2], packed[p / 2 + 3]};
                __builtin_amdgcn_raw_buffer_store_b128(t, obuf, off, 0, 0);
              } else if (SV == 4) {
                const u32x2 t = {packed[p / 2], packed[p / 2 + 1]};
                __builtin_amdgcn_raw_buffer_store_b64(t, obuf, off, 0, 0);
              } else if (SV == 2) {
                __builtin_amdgcn_raw_buffer_store_b32(packed[p / 2], obuf, off, 0, 0);
              } else {
                const unsigned pair = packed[p / 2];
                __builtin_amdgcn_raw_buffer_store_b16(
                    (unsigned short)((p & 1) ? (pair >> 16) : (pair & 0xffffu)), obuf, off, 0, 0);
              }
            }
          }
        }
        // running (max, sum) of the row over this lane's share of the columns
        if (ragged) {
#pragma unroll
          for (int e = 0; e < 16; ++e) y[e] = (vs + e < V) ? y[e] : OT_NEG_INF;
        }
        float tmax = y[0];
#pragma unroll
        for (int e = 1; e < 16; ++e) tmax = fmaxf(tmax, y[e]);
        const float nm = fmaxf(m_run[rs], tmax);
        const float ref = __builtin_isinf(nm) ? 0.f : nm;
        const float oldref = __builtin_isinf(m_run[rs]) ? 0.f : m_run[rs];
        float s = (s_run[rs] == 0.f) ? 0.f : s_run[rs] * exp_fast(oldref - ref);
#pragma unroll
        for (int e = 0; e < 16; ++e) s += exp_fast(y[e] - ref);
        s_run[rs] = s;
        m_run[rs] = nm;
      }
    }
  }

  // a row's two lanes (c, c + 32) merge their halves; the lower one writes
#pragma unroll
  for (int rs = 0; rs < 2; ++rs) {
    const float m2 = __shfl_xor(m_run[rs], 32, kWave), s2 = __shfl_xor(s_run[rs], 32, kWave);
    const float nm = fmaxf(m_run[rs], m2);
    const float ref = __builtin_isinf(nm) ? 0.f : nm;
    const float r1 = __builtin_isinf(m_run[rs]) ? 0.f : m_run[rs];
    const float r2 = __builtin_isinf(m2) ? 0.f : m2;
    const float s = ((s_run[rs] == 0.f) ? 0.f : s_run[rs] * exp_fast(r1 - ref)) +
                    ((s2 == 0.f) ? 0.f : s2 * exp_fast(r2 - ref));
    const unsigned r = (unsigned)(64 * wave + 32 * rs + c);
    if (h == 0 && r < nrows) den[row0 + r] = logf(s) + ref;
  }
}

// lp = (logits[row, blank], logits[row, target]) - den[row] for denominators that
// are already known (cpu.cc:52-100 without its log-sum-exp); T = float or a 2-byte type
template <class E, bool IS_F32>
__global__ __launch_bounds__(kBlock) void gather_given_den_kernel(
    const void *__restrict__ logits, const float *__restrict__ den,
    const int32_t *__restrict__ targets, const int32_t *__restrict__ target_lengths,
    const int32_t *__restrict__ row_splits, int N, int targets_cols, int V, int blank,
    float *__restrict__ lp) {
  const int64_t lattice_rows = row_splits[N];
  const int64_t row = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (row >= lattice_rows) return;
  auto value = [&](int col) -> float {
    const int64_t i = row * (int64_t)V + col;
    if (IS_F32) return static_cast<const float *>(logits)[i];
    return to_float<E>(static_cast<const unsigned short *>(logits)[i]);
  };
  const float d = den[row];
  const float bl = value(blank) - d;
  const int b = find_utterance(row_splits, N, row);
  const int U = target_lengths[b];
  const int u = (int)(row - row_splits[b]) % (U + 1 > 0 ? U + 1 : 1);
  float sym = OT_NEG_INF;
  if (u < U && u < targets_cols) {
    const int col = targets[(int64_t)b * targets_cols + u];
    if ((unsigned)col < (unsigned)V) sym = value(col) - d;
  }
  reinterpret_cast<float2 *>(lp)[row] = make_float2(bl, sym);
}

static inline int launch_status() { return (int)hipGetLastError(); }

template <class E, bool OUT_F32>
static int launch_project(const unsigned short *x, const unsigned short *w, const float *bias,
                          int64_t rows, int32_t D, int32_t V, void *logits, float *den,
                          hipStream_t s) {
  const int64_t blocks = (rows + kProjRows - 1) / kProjRows;
  if (blocks > INT32_MAX) return OT_E_BAD_ARG;
  const unsigned esize = OUT_F32 ? 4u : 2u;
  int sv = (int)(16u / esize);  // elements per store
  while (sv > 1 && (V % sv != 0 || (reinterpret_cast<uintptr_t>(logits) & (uintptr_t)(sv * esize - 1))))
    sv >>= 1;
#define OT_LAUNCH_PROJ(SV_)                                                                       \
  hipLaunchKernelGGL((joiner_project_kernel<E, OUT_F32, SV_>), dim3((unsigned)blocks), dim3(256), \
                     0, s, x, w, bias, rows, D, V, logits, den)
  switch (sv) {
    case 8: if constexpr (!OUT_F32) { OT_LAUNCH_PROJ(8); } break;
    case 4: OT_LAUNCH_PROJ(4); break;
    case 2: OT_LAUNCH_PROJ(2); break;
    default: OT_LAUNCH_PROJ(1); break;
  }
#undef OT_LAUNCH_PROJ
  return launch_status();
}

}  // namespace ot

using namespace ot;

extern "C" {

int ot_joiner_project(const void *x, const void *weight, const float *bias, int32_t dtype,
                      int64_t rows, int32_t D, int32_t V, void *logits, int32_t logits_dtype,
                      float *den, void *stream) {
  if (!x || !weight || !logits || !den || rows <= 0 || rows > INT32_MAX || D <= 0 || V <= 0 ||
      (dtype != OT_DTYPE_F16 && dtype != OT_DTYPE_BF16) ||
      (logits_dtype != OT_DTYPE_F32 && logits_dtype != dtype))
    return OT_E_BAD_ARG;
  // one stage is 32 k-values; offsets inside a workgroup's rows and inside W are 32-bit
  if (D % kProjK != 0 || (int64_t)V * D * 2 > (int64_t)UINT32_MAX ||
      (int64_t)kProjRows * V * 4 > (int64_t)UINT32_MAX || (int64_t)kProjRows * D * 2 > (int64_t)UINT32_MAX)
    return OT_E_BAD_ARG;
  if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(weight) & 15) ||
      (reinterpret_cast<uintptr_t>(bias) & 15) || (reinterpret_cast<uintptr_t>(den) & 3) ||
      (reinterpret_cast<uintptr_t>(logits) & (logits_dtype == OT_DTYPE_F32 ? 3 : 1)))
    return OT_E_MISALIGNED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned short *xp = static_cast<const unsigned short *>(x);
  const unsigned short *wp = static_cast<const unsigned short *>(weight);
  if (dtype == OT_DTYPE_BF16)
    return logits_dtype == OT_DTYPE_F32
               ? launch_project<BF16, true>(xp, wp, bias, rows, D, V, logits, den, s)
               : launch_project<BF16, false>(xp, wp, bias, rows, D, V, logits, den, s);
  return logits_dtype == OT_DTYPE_F32
             ? launch_project<F16, true>(xp, wp, bias, rows, D, V, logits, den, s)
             : launch_project<F16, false>(xp, wp, bias, rows, D, V, logits, den, s);
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
  const dim3 grid((unsigned)((rows + kBlock - 1) / kBlock));
#define OT_LAUNCH_GGD(E_, F32_)                                                                   \
  hipLaunchKernelGGL((gather_given_den_kernel<E_, F32_>), grid, dim3(kBlock), 0, s, logits, den,  \
                     targets, target_lengths, row_splits, N, targets_cols, V, blank, lp)
  if (dtype == OT_DTYPE_F32) OT_LAUNCH_GGD(BF16, true);
  else if (dtype == OT_DTYPE_F16) OT_LAUNCH_GGD(F16, false);
  else OT_LAUNCH_GGD(BF16, false);
#undef OT_LAUNCH_GGD
  return launch_status();
}

}  // extern "C"
