// Packed joiner input for the transducer loss, and its gradient (gfx950).
//
// The loss takes the joiner output for the valid (t, u) cells only, utterances
// concatenated: row_splits[b] + t*(U_b+1) + u.  The reference leaves building
// the joiner's *input* in that layout to the caller and shows it with Python
// lists (README.md:166-177):
//     x = cat([ (enc[b,:T_b].unsqueeze(1) + dec[b,:U_b+1].unsqueeze(0)).reshape(-1, D) ])
//     activation = tanh(x)
// The kernels here do the same from the padded encoder / decoder outputs in one
// pass each way:
//   joiner_pack_kernel         out[row] = act(enc[b,t] + dec[b,u]); write-bound
//   joiner_unpack_grad_kernel  one pass over d(out): complete sums over u for
//                              the encoder, sums over 16 frames for the decoder
//   joiner_dec_reduce_kernel   adds the per-16-frame partial sums, fixed order
// Sums are taken in a fixed order, so results are the same bits on every run.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ot_device.hip.h"
#include "ot_transducer.h"

namespace ot {

// tanh with a relative error of a few ulp over the whole range: the odd series
// below |x| = 0.25 (where 1 - e^-2|x| cancels), the exponential form elsewhere.
__device__ __forceinline__ float tanh_dev(float x) {
  const float ax = __builtin_fabsf(x);
  const float x2 = x * x;
  // x - x^3/3 + 2x^5/15 - 17x^7/315 + 62x^9/2835; next term 1382x^11/155925 < 1e-8 * x at 0.25.
  // Fused multiply-adds written out: the build keeps contraction off.
  float p = __builtin_fmaf(x2, 0.021869488f, -0.053968254f);
  p = __builtin_fmaf(x2, p, 0.13333334f);
  p = __builtin_fmaf(x2, p, -0.333333343f);
  const float small = __builtin_fmaf(x * x2, p, x);
  const float e = __builtin_amdgcn_exp2f(ax * -2.88539004325866699219f);  // exp(-2|x|)
  const float big = __builtin_copysignf((1.f - e) * __builtin_amdgcn_rcpf(1.f + e), x);
  return ax < 0.25f ? small : big;
}

template <int ACT>
__device__ __forceinline__ float activate(float s) {
  return ACT == OT_ACT_TANH ? tanh_dev(s) : ACT == OT_ACT_RELU ? fmaxf(s, 0.f) : s;
}

// tanh for a result that is rounded to 8 or 11 significant bits afterwards:
// 1 - 2 / (1 + e^2|x|), whose absolute error of 1e-7 is below 2^-13 of the result
// from |x| = 4e-4 on; below that tanh(x) = x to 5e-8.  Half the instructions of
// tanh_dev, which is what the 16-bit pack kernel is bound by.
__device__ __forceinline__ float tanh_16bit(float x) {
  const float ax = __builtin_fabsf(x);
  const float e = __builtin_amdgcn_exp2f(ax * 2.88539004325866699219f);  // exp(2|x|), inf is fine
  const float t = __builtin_fmaf(-2.f, __builtin_amdgcn_rcpf(1.f + e), 1.f);
  return ax < 4e-4f ? x : __builtin_copysignf(t, x);
}
template <int ACT>
__device__ __forceinline__ float activate_16bit(float s) {
  return ACT == OT_ACT_TANH ? tanh_16bit(s) : ACT == OT_ACT_RELU ? fmaxf(s, 0.f) : s;
}
// d act(s) / d s
template <int ACT>
__device__ __forceinline__ float activate_slope(float s) {
  if (ACT == OT_ACT_TANH) {
    // 1 - tanh^2 = 4e / (1 + e)^2 with e = exp(-2|s|): no cancellation near |tanh| = 1
    const float e = __builtin_amdgcn_exp2f(__builtin_fabsf(s) * -2.88539004325866699219f);
    const float r = __builtin_amdgcn_rcpf(1.f + e);
    return 4.f * e * (r * r);
  }
  if (ACT == OT_ACT_RELU) return s > 0.f ? 1.f : 0.f;  // 0 at s = 0, like torch.relu's backward
  return 1.f;
}

// ---------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------
// One workgroup = utterance b, kPackFrames frames, kPackPositions positions u,
// up to 256 column units.  A thread keeps its columns of the frames' encoder rows
// in registers and walks u: one decoder load serves kPackFrames output rows, no
// index array is read, and every store instruction of a wave writes a contiguous
// piece of one output row.
constexpr int kPackPositions = 16;  // positions u per workgroup: fastest of 8, 16, 32, 64, all
constexpr int kPackFrames = 2;  // fastest of 1, 2, 4, 8 on MI355X

template <int VEC, int ACT>
__global__ __launch_bounds__(kBlock) void joiner_pack_kernel(
    const float *__restrict__ enc, const float *__restrict__ dec,
    const int32_t *__restrict__ logit_lengths, const int32_t *__restrict__ target_lengths,
    const int32_t *__restrict__ row_splits, int t_stride, int u_stride, int D,
    float *__restrict__ out) {
  const int b = blockIdx.z;
  const int t0 = blockIdx.y * kPackFrames;
  const int T = min(logit_lengths[b], t_stride);
  if (t0 >= T) return;
  const int U1 = min(target_lengths[b] + 1, u_stride);
  const int nvec = D / VEC;
  const int cpb = min(nvec, kBlock);  // column units per workgroup
  const int phases = kBlock / cpb;    // positions u in flight per workgroup
  const int phase = threadIdx.x / cpb;
  const int nslabs = (nvec + cpb - 1) / cpb;
  const int uc = blockIdx.x / nslabs, slab = blockIdx.x - uc * nslabs;
  const int u_begin = uc * kPackPositions, u_end = min(U1, u_begin + kPackPositions);
  const int unit = slab * cpb + (threadIdx.x - phase * cpb);
  if (phase >= phases || unit >= nvec || u_begin >= U1) return;
  const int col = unit * VEC;
  const int nt = min(kPackFrames, T - t0);
  Vec<VEC> e[kPackFrames];
#pragma unroll
  for (int i = 0; i < kPackFrames; ++i) {
#pragma unroll
    for (int k = 0; k < VEC; ++k) e[i].v[k] = 0.f;
    if (i < nt) e[i].load_cached(enc + ((int64_t)(b * t_stride + t0 + i) * D + col));
  }
  float *o = out + (((int64_t)row_splits[b] + (int64_t)t0 * U1) * D + col);
  const float *dp = dec + ((int64_t)b * u_stride * D + col);
  const int64_t frame_stride = (int64_t)U1 * D;
  Vec<VEC> d;
  if (u_begin + phase < u_end) d.load_cached(dp + (int64_t)(u_begin + phase) * D);
  for (int u = u_begin + phase; u < u_end; u += phases) {
    Vec<VEC> dn = d;
    if (u + phases < u_end) dn.load_cached(dp + (int64_t)(u + phases) * D);
#pragma unroll
    for (int i = 0; i < kPackFrames; ++i) {
      if (i < nt) {
        Vec<VEC> y;
#pragma unroll
        for (int k = 0; k < VEC; ++k) y.v[k] = activate<ACT>(e[i].v[k] + d.v[k]);
        y.store_stream(o + (i * frame_stride + (int64_t)u * D));
      }
    }
    d = dn;
  }
}

// The same with 2-byte output (float32 inputs and arithmetic, rounded to nearest
// even): for a joiner whose projection runs in float16 / bfloat16, instead of a
// float32 pack followed by a cast pass.  8 columns per thread, so that a thread
// stores 16 bytes and a wave a contiguous 1 KiB.  With tanh this kernel is bound
// by its arithmetic, not its stores: 8 frames per workgroup (fastest of 2, 8, 16
// at 4, 8 and 16 positions) spread the decoder loads and the index arithmetic
// over four times as many outputs as the float32 kernel's 2.
constexpr int kPackHalfFrames = 8;
template <int ACT, class E>
__global__ __launch_bounds__(kBlock) void joiner_pack_half_kernel(
    const float *__restrict__ enc, const float *__restrict__ dec,
    const int32_t *__restrict__ logit_lengths, const int32_t *__restrict__ target_lengths,
    const int32_t *__restrict__ row_splits, int t_stride, int u_stride, int D,
    unsigned short *__restrict__ out) {
  constexpr int VEC = 8;
  const int b = blockIdx.z;
  const int t0 = blockIdx.y * kPackHalfFrames;
  const int T = min(logit_lengths[b], t_stride);
  if (t0 >= T) return;
  const int U1 = min(target_lengths[b] + 1, u_stride);
  const int nvec = D / VEC;
  const int cpb = min(nvec, kBlock);  // column units per workgroup
  const int phases = kBlock / cpb;    // positions u in flight per workgroup
  const int phase = threadIdx.x / cpb;
  const int nslabs = (nvec + cpb - 1) / cpb;
  const int uc = blockIdx.x / nslabs, slab = blockIdx.x - uc * nslabs;
  const int u_begin = uc * kPackPositions, u_end = min(U1, u_begin + kPackPositions);
  const int unit = slab * cpb + (threadIdx.x - phase * cpb);
  if (phase >= phases || unit >= nvec || u_begin >= U1) return;
  const int col = unit * VEC;
  const int nt = min(kPackHalfFrames, T - t0);
  Vec<4> e[kPackHalfFrames][2];
#pragma unroll
  for (int i = 0; i < kPackHalfFrames; ++i)
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
      for (int k = 0; k < 4; ++k) e[i][p].v[k] = 0.f;
      if (i < nt) e[i][p].load_cached(enc + ((int64_t)(b * t_stride + t0 + i) * D + col + 4 * p));
    }
  unsigned short *o = out + (((int64_t)row_splits[b] + (int64_t)t0 * U1) * D + col);
  const float *dp = dec + ((int64_t)b * u_stride * D + col);
  const int64_t frame_stride = (int64_t)U1 * D;
  Vec<4> d[2];
  if (u_begin + phase < u_end) {
    d[0].load_cached(dp + (int64_t)(u_begin + phase) * D);
    d[1].load_cached(dp + (int64_t)(u_begin + phase) * D + 4);
  }
  for (int u = u_begin + phase; u < u_end; u += phases) {
    Vec<4> dn[2] = {d[0], d[1]};
    if (u + phases < u_end) {
      dn[0].load_cached(dp + (int64_t)(u + phases) * D);
      dn[1].load_cached(dp + (int64_t)(u + phases) * D + 4);
    }
#pragma unroll
    for (int i = 0; i < kPackHalfFrames; ++i) {
      if (i < nt) {
        u32x4 y;
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            const unsigned short lo = from_float<E>(activate_16bit<ACT>(e[i][p].v[2 * k] + d[p].v[2 * k]));
            const unsigned short hi = from_float<E>(activate_16bit<ACT>(e[i][p].v[2 * k + 1] + d[p].v[2 * k + 1]));
            y[2 * p + k] = (unsigned)lo | ((unsigned)hi << 16);
          }
        __builtin_nontemporal_store(y, reinterpret_cast<u32x4 *>(o + (i * frame_stride + (int64_t)u * D)));
      }
    }
    d[0] = dn[0];
    d[1] = dn[1];
  }
}

// ---------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------
constexpr int kTileFrames = OT_JOINER_TILE_FRAMES;  // frames per workgroup
constexpr int kSlabLanes = 16;      // lanes across the columns of a slab: 16 x 16 bytes of a float32 row,
constexpr int kSlabLanesHalf = 32;  // 32 x 8 bytes of a 2-byte row (256 contiguous bytes either way)

// One workgroup: utterance b = blockIdx.z, frames [t0, t0 + 16), columns
// [slab*SL*VEC, (slab+1)*SL*VEC).  Thread (phase, half, lane): columns lane*VEC.., the
// positions u = phase, phase + P, ... and 8 of the tile's 16 frames.  For one u it loads
// its 8 frames' values (8 independent loads), adds them up for the decoder (the two
// halves meet through one cross-lane exchange) and into 8 per-frame accumulators for
// the encoder.  The encoder sums of the workgroup's threads are then added through
// DPP/LDS in a fixed order.
// VEC elements of the incoming gradient: float32 (G = float) or a 2-byte type.  Loading
// and widening are two steps so that a thread's 16 loads are all issued before the
// first value is used.
template <class G, int VEC> struct GradIO {
  typedef unsigned short raw_t __attribute__((ext_vector_type(VEC == 4 ? 4 : 2)));
  static __device__ __forceinline__ raw_t load(const void *base, int64_t index) {
    const unsigned short *p = static_cast<const unsigned short *>(base) + index;
    raw_t r;
    if (VEC == 4) {
      r = *reinterpret_cast<const raw_t *>(p);
    } else {
      r[0] = *p;
      r[1] = 0;
    }
    return r;
  }
  static __device__ __forceinline__ void widen(raw_t r, Vec<VEC> &g) {
#pragma unroll
    for (int k = 0; k < VEC; ++k) g.v[k] = to_float<G>(r[k]);
  }
};
template <int VEC> struct GradIO<float, VEC> {
  typedef Vec<VEC> raw_t;
  static __device__ __forceinline__ raw_t load(const void *base, int64_t index) {
    raw_t r;
    r.load(static_cast<const float *>(base) + index);
    return r;
  }
  static __device__ __forceinline__ void widen(const raw_t &r, Vec<VEC> &g) { g = r; }
};

// G: element type of grad_out (float, F16 or BF16); everything else is float32.
//
// Thread (phase, half, lane): columns lane*VEC.., the positions u = phase, phase + P, ...
// (P = 128 / SL phases per workgroup), and the 8 frames half*8 .. half*8+7 of the tile.
// The two halves of a position sit in one wave, SL lanes apart, and meet through one
// cross-lane exchange per position.  With all 16 frames in one thread the kernel needs
// 170-250 registers (16 values in flight, 16 accumulators, 16 addresses), i.e. two
// waves per SIMD, and spends its time waiting: half as many frames per thread and twice
// the waves keep as many loads in flight and overlap them with the arithmetic.
constexpr int kHalfFrames = kTileFrames / 2;

template <int VEC, int ACT, class G, int SL>
__global__ __launch_bounds__(kBlock) void joiner_unpack_grad_kernel(
    const void *__restrict__ grad_out, const float *__restrict__ enc,
    const float *__restrict__ dec, const int32_t *__restrict__ logit_lengths,
    const int32_t *__restrict__ target_lengths, const int32_t *__restrict__ row_splits,
    int t_stride, int u_stride, int D, float *__restrict__ grad_enc,
    float *__restrict__ dec_partial) {
  static_assert(2 * SL <= kWave, "both halves of a position in one wave");
  constexpr int kPhases = kBlock / (2 * SL);
  __shared__ __attribute__((aligned(16))) float s_enc[kTileFrames][SL * VEC];
  __shared__ __attribute__((aligned(16))) float s_red[kWavesPerBlock][kTileFrames][SL * VEC];
  const int b = blockIdx.z;
  const int t0 = blockIdx.y * kTileFrames;
  const int lane = threadIdx.x & (SL - 1);
  const int half = (threadIdx.x / SL) & 1;
  const int phase = threadIdx.x / (2 * SL);
  const int col = (blockIdx.x * SL + lane) * VEC;
  const bool col_ok = col < D;  // D is a multiple of VEC
  const int T = min(logit_lengths[b], t_stride);
  const int U1 = min(target_lengths[b] + 1, u_stride);
  const int64_t row0 = row_splits[b];
  const int ntiles = gridDim.y;

  // frames of this tile that exist; the rest of the tile (padding of the encoder
  // output) gets zeros
  const int nframes = max(0, min(kTileFrames, T - t0));
  if (ACT != OT_ACT_NONE) {
    for (int i = threadIdx.x / SL; i < kTileFrames; i += (kBlock / SL)) {
      Vec<VEC> e;
#pragma unroll
      for (int k = 0; k < VEC; ++k) e.v[k] = 0.f;
      if (i < nframes && col_ok) e.load_cached(enc + ((int64_t)(b * t_stride + t0 + i) * D + col));
      e.store_lds(&s_enc[i][lane * VEC]);
    }
    __syncthreads();
  }

  Vec<VEC> acc[kHalfFrames];
#pragma unroll
  for (int i = 0; i < kHalfFrames; ++i)
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc[i].v[k] = 0.f;

  if (nframes > 0 && col_ok) {
    const int64_t frame_stride = (int64_t)U1 * D;
    const int f0 = half * kHalfFrames;  // this thread's first frame of the tile
    for (int u = phase; u < U1; u += kPhases) {
      const int64_t p = (row0 + (int64_t)t0 * U1 + u) * D + col;
      // frames past the tile's last one re-read frame 0 and are zeroed afterwards: no
      // branch between the loads
      typename GradIO<G, VEC>::raw_t raw[kHalfFrames];
#pragma unroll
      for (int i = 0; i < kHalfFrames; ++i)
        raw[i] = GradIO<G, VEC>::load(grad_out, p + (f0 + i < nframes ? f0 + i : 0) * frame_stride);
      Vec<VEC> d, sum;
#pragma unroll
      for (int k = 0; k < VEC; ++k) sum.v[k] = 0.f;
      if (ACT != OT_ACT_NONE) d.load_cached(dec + ((int64_t)(b * u_stride + u) * D + col));
#pragma unroll
      for (int i = 0; i < kHalfFrames; ++i) {
        Vec<VEC> g;
        GradIO<G, VEC>::widen(raw[i], g);
        if (f0 + i >= nframes) {
#pragma unroll
          for (int k = 0; k < VEC; ++k) g.v[k] = 0.f;
        }
        if (ACT != OT_ACT_NONE) {
          Vec<VEC> e;
          e.load_lds(&s_enc[f0 + i][lane * VEC]);
#pragma unroll
          for (int k = 0; k < VEC; ++k) g.v[k] *= activate_slope<ACT>(e.v[k] + d.v[k]);
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          sum.v[k] += g.v[k];
          acc[i].v[k] += g.v[k];
        }
      }
      // frames 0-7 + frames 8-15, in that order in both lanes: the same bits as one sum
      // over the halves' sums on every run
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const float other = __shfl_xor(sum.v[k], SL, kWave);
        sum.v[k] = half == 0 ? sum.v[k] + other : other + sum.v[k];
      }
      if (half == 0)
        sum.store(dec_partial + ((((int64_t)b * ntiles + blockIdx.y) * u_stride + u) * D + col));
    }
  }

  // encoder: add the phases of a wave (lanes 2 * SL apart), then the waves
  if (2 * SL < kWave) {
#pragma unroll
    for (int i = 0; i < kHalfFrames; ++i)
#pragma unroll
      for (int k = 0; k < VEC; ++k) acc[i].v[k] += __shfl_xor(acc[i].v[k], 2 * SL, kWave);
  }
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) < 2 * SL) {
#pragma unroll
    for (int i = 0; i < kHalfFrames; ++i)
      acc[i].store_lds(&s_red[wave][half * kHalfFrames + i][lane * VEC]);
  }
  __syncthreads();
  // 16 frames x SL (frame, lane) pairs over the workgroup's threads
  for (int pair = threadIdx.x; pair < kTileFrames * SL; pair += kBlock) {
    const int i = pair / SL, l = pair & (SL - 1);
    const int c = (blockIdx.x * SL + l) * VEC;
    const int t = t0 + i;
    if (t < t_stride && c < D) {
      Vec<VEC> r;
#pragma unroll
      for (int k = 0; k < VEC; ++k) r.v[k] = 0.f;
#pragma unroll
      for (int w = 0; w < kWavesPerBlock; ++w) {
        Vec<VEC> x;
        x.load_lds(&s_red[w][i][l * VEC]);
#pragma unroll
        for (int k = 0; k < VEC; ++k) r.v[k] += x.v[k];
      }
      r.store(grad_enc + ((int64_t)(b * t_stride + t) * D + c));
    }
  }
}

// grad_dec[b,u,:] = sum over the frame tiles of utterance b, in tile order;
// zero for the padding positions u > U_b.
template <int VEC>
__global__ __launch_bounds__(kBlock) void joiner_dec_reduce_kernel(
    const float *__restrict__ dec_partial, const int32_t *__restrict__ logit_lengths,
    const int32_t *__restrict__ target_lengths, int N, int t_stride, int u_stride, int D,
    int ntiles, float *__restrict__ grad_dec) {
  const int nvec = D / VEC;
  const int64_t unit = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t total = (int64_t)N * u_stride * nvec;
  if (unit >= total) return;
  const int c = (int)(unit % nvec) * VEC;
  const int64_t bu = unit / nvec;
  const int u = (int)(bu % u_stride), b = (int)(bu / u_stride);
  Vec<VEC> r;
#pragma unroll
  for (int k = 0; k < VEC; ++k) r.v[k] = 0.f;
  if (u <= target_lengths[b]) {
    const int T = min(logit_lengths[b], t_stride);
    const int used = (T + kTileFrames - 1) / kTileFrames;
    for (int tile = 0; tile < used; ++tile) {
      Vec<VEC> x;
      x.load_cached(dec_partial + ((((int64_t)b * ntiles + tile) * u_stride + u) * D + c));
#pragma unroll
      for (int k = 0; k < VEC; ++k) r.v[k] += x.v[k];
    }
  }
  r.store(grad_dec + (bu * D + c));
}

static inline int launch_status() { return (int)hipGetLastError(); }
static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
static inline bool aligned4(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 3) == 0; }
static inline bool known_activation(int32_t a) {
  return a == OT_ACT_NONE || a == OT_ACT_TANH || a == OT_ACT_RELU;
}

}  // namespace ot

using namespace ot;

extern "C" {

int ot_joiner_pack(const float *enc, const float *dec, const int32_t *logit_lengths,
                   const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                   int32_t t_stride, int32_t u_stride, int32_t D, int32_t activation, float *out,
                   void *stream) {
  if (!enc || !dec || !logit_lengths || !target_lengths || !row_splits || !out || N <= 0 ||
      N > 65535 || t_stride <= 0 || u_stride <= 0 || D <= 0 ||
      (int64_t)N * t_stride > INT32_MAX || (int64_t)N * u_stride > INT32_MAX ||
      !known_activation(activation))
    return OT_E_BAD_ARG;
  if (!aligned4(enc) || !aligned4(dec) || !aligned4(out)) return OT_E_MISALIGNED;
  if ((t_stride + kPackFrames - 1) / kPackFrames > 65535) return OT_E_TOO_LONG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int vec = (D % 4 == 0 && aligned16(enc) && aligned16(dec) && aligned16(out)) ? 4 : 1;
  const int nvec = D / vec;
  const int cpb = nvec < kBlock ? nvec : kBlock;
  const dim3 grid((unsigned)(((nvec + cpb - 1) / cpb) * ((u_stride + kPackPositions - 1) / kPackPositions)),
                  (unsigned)((t_stride + kPackFrames - 1) / kPackFrames), (unsigned)N);
#define OT_LAUNCH_PACKT(VEC_, ACT_)                                                             \
  hipLaunchKernelGGL((joiner_pack_kernel<VEC_, ACT_>), grid, dim3(kBlock), 0, s, enc, dec, \
                     logit_lengths, target_lengths, row_splits, t_stride, u_stride, D, out)
  if (activation == OT_ACT_TANH) {
    if (vec == 4) OT_LAUNCH_PACKT(4, OT_ACT_TANH); else OT_LAUNCH_PACKT(1, OT_ACT_TANH);
  } else if (activation == OT_ACT_RELU) {
    if (vec == 4) OT_LAUNCH_PACKT(4, OT_ACT_RELU); else OT_LAUNCH_PACKT(1, OT_ACT_RELU);
  } else {
    if (vec == 4) OT_LAUNCH_PACKT(4, OT_ACT_NONE); else OT_LAUNCH_PACKT(1, OT_ACT_NONE);
  }
#undef OT_LAUNCH_PACKT
  return launch_status();
}

int ot_joiner_pack_half(const float *enc, const float *dec, const int32_t *logit_lengths,
                        const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                        int32_t t_stride, int32_t u_stride, int32_t D, int32_t activation,
                        int32_t out_dtype, void *out, void *stream) {
  if (!enc || !dec || !logit_lengths || !target_lengths || !row_splits || !out || N <= 0 ||
      N > 65535 || t_stride <= 0 || u_stride <= 0 || D <= 0 || D % 8 != 0 ||
      (int64_t)N * t_stride > INT32_MAX || (int64_t)N * u_stride > INT32_MAX ||
      !known_activation(activation) ||
      (out_dtype != OT_DTYPE_F16 && out_dtype != OT_DTYPE_BF16))
    return OT_E_BAD_ARG;
  if (!aligned16(enc) || !aligned16(dec) || !aligned16(out)) return OT_E_MISALIGNED;
  if ((t_stride + kPackHalfFrames - 1) / kPackHalfFrames > 65535) return OT_E_TOO_LONG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int nvec = D / 8;
  const int cpb = nvec < kBlock ? nvec : kBlock;
  const dim3 grid((unsigned)(((nvec + cpb - 1) / cpb) * ((u_stride + kPackPositions - 1) / kPackPositions)),
                  (unsigned)((t_stride + kPackHalfFrames - 1) / kPackHalfFrames), (unsigned)N);
  unsigned short *o = static_cast<unsigned short *>(out);
#define OT_LAUNCH_PACKH(ACT_, E_)                                                              \
  hipLaunchKernelGGL((joiner_pack_half_kernel<ACT_, E_>), grid, dim3(kBlock), 0, s, enc, dec,  \
                     logit_lengths, target_lengths, row_splits, t_stride, u_stride, D, o)
  if (activation == OT_ACT_TANH) {
    if (out_dtype == OT_DTYPE_F16) OT_LAUNCH_PACKH(OT_ACT_TANH, F16); else OT_LAUNCH_PACKH(OT_ACT_TANH, BF16);
  } else if (activation == OT_ACT_RELU) {
    if (out_dtype == OT_DTYPE_F16) OT_LAUNCH_PACKH(OT_ACT_RELU, F16); else OT_LAUNCH_PACKH(OT_ACT_RELU, BF16);
  } else {
    if (out_dtype == OT_DTYPE_F16) OT_LAUNCH_PACKH(OT_ACT_NONE, F16); else OT_LAUNCH_PACKH(OT_ACT_NONE, BF16);
  }
#undef OT_LAUNCH_PACKH
  return launch_status();
}

size_t ot_joiner_unpack_workspace_bytes(int32_t N, int32_t t_stride, int32_t u_stride, int32_t D) {
  if (N <= 0 || t_stride <= 0 || u_stride <= 0 || D <= 0) return 0;
  const size_t ntiles = ((size_t)t_stride + kTileFrames - 1) / kTileFrames;
  return (size_t)N * ntiles * (size_t)u_stride * (size_t)D * sizeof(float);
}

int ot_joiner_unpack_grad_from(const void *grad_out, int32_t grad_dtype, const float *enc,
                               const float *dec, const int32_t *logit_lengths,
                               const int32_t *target_lengths, const int32_t *row_splits, int32_t N,
                               int32_t t_stride, int32_t u_stride, int32_t D, int32_t activation,
                               void *workspace, size_t workspace_bytes, float *grad_enc,
                               float *grad_dec, void *stream) {
  if (grad_dtype != OT_DTYPE_F32 && grad_dtype != OT_DTYPE_F16 && grad_dtype != OT_DTYPE_BF16)
    return OT_E_BAD_ARG;
  const bool g32 = grad_dtype == OT_DTYPE_F32;
  if (!grad_out || !logit_lengths || !target_lengths || !row_splits || !workspace || !grad_enc ||
      !grad_dec || N <= 0 || N > 65535 || t_stride <= 0 || u_stride <= 0 || D <= 0 ||
      (int64_t)N * t_stride > INT32_MAX || (int64_t)N * u_stride > INT32_MAX ||
      !known_activation(activation) ||
      (activation != OT_ACT_NONE && (!enc || !dec)))
    return OT_E_BAD_ARG;
  if (workspace_bytes < ot_joiner_unpack_workspace_bytes(N, t_stride, u_stride, D))
    return OT_E_BAD_ARG;
  if ((reinterpret_cast<uintptr_t>(grad_out) & (g32 ? 3 : 1)) || !aligned4(enc) || !aligned4(dec) ||
      !aligned4(grad_enc) || !aligned4(grad_dec) || !aligned16(workspace))
    return OT_E_MISALIGNED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // 4 columns per thread need 16-byte (float32) / 8-byte (2-byte types) aligned rows
  const bool v4 = D % 4 == 0 && (reinterpret_cast<uintptr_t>(grad_out) & (g32 ? 15 : 7)) == 0 &&
                  aligned16(grad_enc) && aligned16(grad_dec) &&
                  (activation == OT_ACT_NONE || (aligned16(enc) && aligned16(dec)));
  const int vec = v4 ? 4 : 1;
  const int ntiles = (t_stride + kTileFrames - 1) / kTileFrames;
  if (ntiles > 65535) return OT_E_TOO_LONG;
  const int slab = (g32 ? kSlabLanes : kSlabLanesHalf) * vec;
  const dim3 grid((unsigned)((D + slab - 1) / slab), (unsigned)ntiles, (unsigned)N);
  float *partial = static_cast<float *>(workspace);
#define OT_LAUNCH_UNPACK(VEC_, ACT_, G_, SL_)                                                 \
  hipLaunchKernelGGL((joiner_unpack_grad_kernel<VEC_, ACT_, G_, SL_>), grid, dim3(kBlock), 0, s, \
                     grad_out, enc, dec, logit_lengths, target_lengths, row_splits, t_stride, \
                     u_stride, D, grad_enc, partial)
#define OT_LAUNCH_UNPACK_G(VEC_, ACT_)                                                  \
  if (g32) OT_LAUNCH_UNPACK(VEC_, ACT_, float, kSlabLanes);                             \
  else if (grad_dtype == OT_DTYPE_F16) OT_LAUNCH_UNPACK(VEC_, ACT_, F16, kSlabLanesHalf); \
  else OT_LAUNCH_UNPACK(VEC_, ACT_, BF16, kSlabLanesHalf)
  if (activation == OT_ACT_TANH) {
    if (vec == 4) { OT_LAUNCH_UNPACK_G(4, OT_ACT_TANH); } else { OT_LAUNCH_UNPACK_G(1, OT_ACT_TANH); }
  } else if (activation == OT_ACT_RELU) {
    if (vec == 4) { OT_LAUNCH_UNPACK_G(4, OT_ACT_RELU); } else { OT_LAUNCH_UNPACK_G(1, OT_ACT_RELU); }
  } else {
    if (vec == 4) { OT_LAUNCH_UNPACK_G(4, OT_ACT_NONE); } else { OT_LAUNCH_UNPACK_G(1, OT_ACT_NONE); }
  }
#undef OT_LAUNCH_UNPACK_G
#undef OT_LAUNCH_UNPACK
  int rc = launch_status();
  if (rc) return rc;
  const int64_t units = (int64_t)N * u_stride * (D / vec);
  const int64_t blocks = (units + kBlock - 1) / kBlock;
  if (blocks > INT32_MAX) return OT_E_BAD_ARG;
  if (vec == 4)
    hipLaunchKernelGGL(joiner_dec_reduce_kernel<4>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                       partial, logit_lengths, target_lengths, N, t_stride, u_stride, D, ntiles,
                       grad_dec);
  else
    hipLaunchKernelGGL(joiner_dec_reduce_kernel<1>, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                       partial, logit_lengths, target_lengths, N, t_stride, u_stride, D, ntiles,
                       grad_dec);
  return launch_status();
}

int ot_joiner_unpack_grad(const float *grad_out, const float *enc, const float *dec,
                          const int32_t *logit_lengths, const int32_t *target_lengths,
                          const int32_t *row_splits, int32_t N, int32_t t_stride, int32_t u_stride,
                          int32_t D, int32_t activation, void *workspace, size_t workspace_bytes,
                          float *grad_enc, float *grad_dec, void *stream) {
  return ot_joiner_unpack_grad_from(grad_out, OT_DTYPE_F32, enc, dec, logit_lengths, target_lengths,
                                    row_splits, N, t_stride, u_stride, D, activation, workspace,
                                    workspace_bytes, grad_enc, grad_dec, stream);
}

}  // extern "C"
