// Torch extension `_optimized_transducer`: the drop-in for the reference's
// pybind11 module (optimized_transducer/python/csrc/optimized_transducer.cc:12-19)
// and its argument checks / dispatch (optimized_transducer/csrc/transducer-loss.cc:21-96).
//
// This file only checks arguments, allocates through torch's caching allocator
// and enqueues the C-ABI kernels of include/ot_transducer.h on torch's current
// HIP stream.  There is no CPU implementation behind it: CPU tensors, which the
// reference hands to ComputeTransducerLossCpu (transducer-loss.cc:68-74), are
// checked like the reference checks them, copied to the current HIP device,
// computed there and copied back (the gradient of logits input into the caller's
// logits storage, as cpu.cc:814 aliases it).
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPFunctions.h>
#include <hip/hip_runtime_api.h>
#include <torch/extension.h>

#include <atomic>
#include <cstdlib>
#include <mutex>
#include <sstream>
#include <string>
#include <tuple>
#include <vector>

#include "ot_transducer.h"

namespace {

void check_hip(hipError_t e, const char *file, int line) {
  if (e != hipSuccess) {
    std::ostringstream os;
    os << file << ":" << line << ": " << hipGetErrorString(e) << "\n";
    throw std::runtime_error(os.str());
  }
}
void check_ot(int rc, const char *file, int line) {
  if (rc != 0) {
    std::ostringstream os;
    os << file << ":" << line << ": " << ot_error_string(rc) << "\n";
    throw std::runtime_error(os.str());
  }
}
#define OT_CHECK_HIP(x) check_hip((x), __FILE__, __LINE__)
#define OT_CHECK(x) check_ot((x), __FILE__, __LINE__)

// ---- optional per-kernel timing (hipEvents on the launch stream) ------------
struct Timed {
  std::string name;
  hipEvent_t start, stop;
};
std::mutex g_prof_mutex;
bool g_profiling = false;
std::vector<Timed> g_timed;

struct ScopedTimer {
  hipStream_t stream;
  Timed t;
  bool on;
  ScopedTimer(const char *name, hipStream_t s) : stream(s), on(g_profiling) {
    if (!on) return;
    t.name = name;
    OT_CHECK_HIP(hipEventCreate(&t.start));
    OT_CHECK_HIP(hipEventCreate(&t.stop));
    OT_CHECK_HIP(hipEventRecord(t.start, stream));
  }
  ~ScopedTimer() {
    if (!on) return;
    (void)hipEventRecord(t.stop, stream);
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    g_timed.push_back(t);
  }
};

void set_profiling(bool on) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_profiling = on;
}

// Returns [(kernel name, milliseconds)] recorded since the last call; blocks
// until the recorded events have completed.
std::vector<std::pair<std::string, double>> take_profile() {
  std::vector<Timed> timed;
  {
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    timed.swap(g_timed);
  }
  std::vector<std::pair<std::string, double>> out;
  for (auto &t : timed) {
    float ms = 0.f;
    OT_CHECK_HIP(hipEventSynchronize(t.stop));
    OT_CHECK_HIP(hipEventElapsedTime(&ms, t.start, t.stop));
    out.emplace_back(t.name, (double)ms);
    (void)hipEventDestroy(t.start);
    (void)hipEventDestroy(t.stop);
  }
  return out;
}

// hipEvent owned for the duration of one call (timing disabled)
struct EventGuard {
  hipEvent_t ev = nullptr;
  EventGuard() { OT_CHECK_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming)); }
  ~EventGuard() { (void)hipEventDestroy(ev); }
  EventGuard(const EventGuard &) = delete;
  EventGuard &operator=(const EventGuard &) = delete;
};

// An event recorded behind a kernel that writes into pinned host memory.  Whoever owns
// that memory must not release it while the kernel may still run: if the call unwinds
// (an argument check or a launch throws) before the event has been waited for, the
// destructor waits.  Declare it after the host tensor so that it is destroyed first.
struct HostWriteGuard {
  EventGuard event;
  hipStream_t stream;
  bool recorded = false, waited = false;
  explicit HostWriteGuard(hipStream_t s) : stream(s) {}
  void record() {
    OT_CHECK_HIP(hipEventRecord(event.ev, stream));
    recorded = true;
  }
  void wait() {
    OT_CHECK_HIP(hipEventSynchronize(event.ev));
    waited = true;
  }
  ~HostWriteGuard() {
    if (waited) return;
    // unwinding: the kernel may have been launched even if the event was not recorded
    if (recorded) (void)hipEventSynchronize(event.ev);
    else (void)hipStreamSynchronize(stream);
  }
};

// Batches below this many logits elements run on one stream.
constexpr int64_t kOverlapMinElements = (int64_t)32 << 20;

// The two-stream schedule is opt-in (set_overlap(true) or OT_TRANSDUCER_OVERLAP=1):
// on MI355X the lattice kernel slows down about five-fold when it shares the
// memory system with a streaming kernel, which costs more than the overlap saves
// (0.93 ms against 0.85 ms per step at N=32, V=500).
std::atomic<int> g_overlap{-1};
bool overlap_enabled() {
  int v = g_overlap.load();
  if (v < 0) {
    const char *e = std::getenv("OT_TRANSDUCER_OVERLAP");
    v = (e && e[0] == '1') ? 1 : 0;
    g_overlap.store(v);
  }
  return v == 1;
}
void set_overlap(bool on) { g_overlap.store(on ? 1 : 0); }

// ---- the value checks of transducer-loss.cc:49-66, given the batch facts ----
void check_batch_values(const torch::Tensor &logits, const torch::Tensor &targets,
                        int64_t sum_all_TU, int64_t targets_max, int64_t target_len_max,
                        int32_t blank) {
  torch::CheckedFrom checked_from = "ComputeTransducerLoss";
  torch::checkSize(checked_from, torch::TensorArg(logits, "logits", 0), 0, sum_all_TU);
  TORCH_CHECK(targets_max < logits.size(1), "targets.max() vs logits.size(1) is ", targets_max,
              " vs ", logits.size(1), ". Expect targets.max() < logits.size(1)");
  TORCH_CHECK((0 <= blank && blank < logits.size(1)), "blank vs logits.size(1) is ", blank,
              " vs ", logits.size(1), ". Expect 0 <= blank < logits.size(1)");
  TORCH_CHECK((targets.size(1) == target_len_max),
              "targets.size(1) should be equal to target_lengths.max().",
              "But targets.size(1) is ", targets.size(1), ", and target_lengths.max() is ",
              target_len_max);
}

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// OT_DTYPE_F16 / OT_DTYPE_BF16 for half-precision logits, OT_DTYPE_F32 for anything else
inline int half_dtype(const torch::Tensor &t) {
  if (t.scalar_type() == torch::kHalf) return OT_DTYPE_F16;
  if (t.scalar_type() == torch::kBFloat16) return OT_DTYPE_BF16;
  return OT_DTYPE_F32;
}

// With `denominators` given (the per-row log-sum-exp of logits input, as
// joiner_project produces them), the pass over the logits for them is skipped.
// With `coefficients` set, the (rows, V) gradient pass is left to
// apply_deferred_gradient: the per-row coefficients go into a tensor of their own,
// handed back through the pointer, and the returned gradient is None.
// With `reduced_loss` set, the 0-dim loss -grad_scale * scores.sum() is computed as
// well: by the row-coefficient launch where there is one, else by a launch of its own.
std::pair<torch::Tensor, torch::optional<torch::Tensor>> compute_impl(
    torch::Tensor &logits, const torch::Tensor &targets, const torch::Tensor &logit_lengths,
    const torch::Tensor &target_lengths, int32_t blank, bool from_log_softmax,
    bool one_sym_per_frame, double grad_scale, torch::Tensor *coefficients,
    const torch::optional<torch::Tensor> &denominators = torch::nullopt,
    torch::Tensor *reduced_loss = nullptr) {
  const bool defer = coefficients != nullptr;
  const bool have_den = denominators.has_value() && denominators->defined();
  auto logits_arg = torch::TensorArg(logits, "logits", 0);
  auto targets_arg = torch::TensorArg(targets, "targets", 1);
  auto logit_lengths_arg = torch::TensorArg(logit_lengths, "logit_lengths", 2);
  auto target_lengths_arg = torch::TensorArg(target_lengths, "target_lengths", 3);
  torch::CheckedFrom checked_from = "ComputeTransducerLoss";

  // transducer-loss.cc:33-46, same order
  // float32 as in the reference; float16 / bfloat16 logits are an addition (the
  // two passes over (rows, V) then read 2-byte elements, everything else is float32)
  const int dtype = half_dtype(logits);
  if (dtype == OT_DTYPE_F32) torch::checkScalarType(checked_from, logits_arg, torch::kFloat);
  torch::checkScalarType(checked_from, targets_arg, torch::kInt32);
  torch::checkScalarType(checked_from, logit_lengths_arg, torch::kInt32);
  torch::checkScalarType(checked_from, target_lengths_arg, torch::kInt32);
  torch::checkAllContiguous(checked_from,
                            {logits_arg, targets_arg, logit_lengths_arg, target_lengths_arg});
  torch::checkDim(checked_from, logits_arg, 2);
  torch::checkDim(checked_from, targets_arg, 2);
  torch::checkDim(checked_from, logit_lengths_arg, 1);
  torch::checkDim(checked_from, target_lengths_arg, 1);
  torch::checkSameSize(checked_from, logit_lengths_arg, target_lengths_arg);

  const int64_t N = logit_lengths.size(0);
  const int64_t rows = logits.size(0);
  const int64_t V = logits.size(1);
  const int64_t S = targets.size(1);

  if (logits.device().type() == torch::kCPU) {
    // Same checks as the reference makes before it dispatches on the device
    // (transducer-loss.cc:49-71), on the host tensors.
    TORCH_CHECK(N > 0, "logit_lengths must not be empty");
    const int64_t sum_all_TU =
        (logit_lengths.to(torch::kLong) * (target_lengths.to(torch::kLong) + 1)).sum().item<int64_t>();
    const int64_t targets_max = targets.numel() ? targets.max().item<int32_t>() : INT32_MIN;
    const int64_t target_len_max = target_lengths.max().item<int32_t>();
    check_batch_values(logits, targets, sum_all_TU, targets_max, target_len_max, blank);
    torch::checkDeviceType(checked_from, {logits, targets, logit_lengths, target_lengths},
                           torch::kCPU);
    TORCH_CHECK(!defer, "defer_gradient needs logits on a HIP device");
    TORCH_CHECK(!have_den || denominators->device().type() == torch::kCPU,
                "denominators must be on the device of logits");
    // The reference computes these on the host (ComputeTransducerLossCpu, cpu.cc:754-827).
    // This build computes on the GPU only: stage the batch through the current HIP device.
    if (!torch::cuda::is_available())
      throw std::runtime_error(
          "optimized_transducer_amd: CPU tensors are computed on a HIP device (there is no CPU "
          "implementation), and no HIP device is available");
    const torch::Device dev(torch::kCUDA, c10::hip::current_device());
    torch::Tensor dev_logits = logits.detach().to(dev);
    if (logits.requires_grad()) dev_logits.requires_grad_(true);
    torch::optional<torch::Tensor> dev_den;
    if (have_den) dev_den = denominators->to(dev);
    torch::Tensor dev_loss;
    auto out = compute_impl(dev_logits, targets.to(dev), logit_lengths.to(dev),
                            target_lengths.to(dev), blank, from_log_softmax, one_sym_per_frame,
                            grad_scale, nullptr, dev_den, reduced_loss ? &dev_loss : nullptr);
    if (reduced_loss) *reduced_loss = dev_loss.cpu();
    torch::Tensor scores = out.first.cpu();
    if (!out.second.has_value()) return {scores, torch::nullopt};
    // cpu.cc:803: a new tensor for log-softmax input
    if (from_log_softmax) return {scores, out.second->cpu()};
    // cpu.cc:814: for logits input the gradient IS the caller's logits buffer
    logits.detach().copy_(*out.second);
    return {scores, logits};
  }

  torch::checkAllSameGPU(checked_from,
                         {logits_arg, targets_arg, logit_lengths_arg, target_lengths_arg});
  TORCH_CHECK(N > 0, "logit_lengths must not be empty");
  TORCH_CHECK(targets.size(0) == N, "targets.size(0) is ", targets.size(0),
              " but there are ", N, " utterances");
  TORCH_CHECK(rows > 0 && V > 0, "logits must not be empty");
  TORCH_CHECK(rows <= INT32_MAX && N < INT32_MAX && V <= INT32_MAX && S < OT_MAX_U1,
              "tensor sizes exceed what 32-bit row offsets can address");
  if (have_den) {
    TORCH_CHECK(!from_log_softmax, "denominators belong to logits input (from_log_softmax=False)");
    TORCH_CHECK(denominators->scalar_type() == torch::kFloat && denominators->dim() == 1 &&
                    denominators->size(0) == rows && denominators->is_contiguous() &&
                    denominators->device() == logits.device(),
                "denominators must be a contiguous float32 tensor of shape (logits.size(0),) on "
                "the device of logits");
  }

  c10::hip::HIPGuardMasqueradingAsCUDA device_guard(logits.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();

  // workspace: row_splits | scores_beta | den | lp | alpha | beta | row coefficients
  const size_t off_sbeta = align256((N + 1) * sizeof(int32_t));
  const size_t off_den = off_sbeta + align256(N * sizeof(float));
  const size_t off_lp = off_den + align256(rows * sizeof(float));
  const size_t off_alpha = off_lp + align256(rows * 2 * sizeof(float));
  const size_t off_beta = off_alpha + align256(rows * sizeof(float));
  const size_t off_coef = off_beta + align256(rows * sizeof(float));
  const size_t total = off_coef + (defer ? 0 : align256(ot_gradient_scratch_bytes(rows)));
  torch::Tensor workspace =
      torch::empty({(int64_t)total}, logits.options().dtype(torch::kUInt8));
  char *w = static_cast<char *>(workspace.data_ptr());
  char *coef = w + off_coef;
  if (defer && logits.requires_grad()) {
    // outlives this call, unlike the rest of the workspace
    *coefficients = torch::empty({(int64_t)ot_gradient_scratch_bytes(rows)},
                                 logits.options().dtype(torch::kUInt8));
    coef = static_cast<char *>(coefficients->data_ptr());
  }
  auto *row_splits = reinterpret_cast<int32_t *>(w);
  auto *scores_beta = reinterpret_cast<float *>(w + off_sbeta);
  auto *den = have_den ? denominators->data_ptr<float>() : reinterpret_cast<float *>(w + off_den);
  auto *lp = reinterpret_cast<float *>(w + off_lp);
  auto *alpha = reinterpret_cast<float *>(w + off_alpha);
  auto *beta = reinterpret_cast<float *>(w + off_beta);

  const void *p_logits = logits.data_ptr();
  const float *p_logits32 = dtype == OT_DTYPE_F32 ? logits.data_ptr<float>() : nullptr;
  const int32_t *p_targets = S > 0 ? targets.data_ptr<int32_t>() : nullptr;
  const int32_t *p_T = logit_lengths.data_ptr<int32_t>();
  const int32_t *p_U = target_lengths.data_ptr<int32_t>();

  // One device pass gathers every fact the checks need and writes them, and a
  // copy of row_splits, straight into pinned host memory; one event wait
  // replaces the reference's blocking .item() calls (transducer-loss.cc:49,53,62
  // and cuda.cu:166,169,242,245).
  const size_t host_splits_off = align256(sizeof(ot_batch_status));
  torch::Tensor status_host = torch::empty(
      {(int64_t)(host_splits_off + (N + 1) * sizeof(int32_t))},
      torch::TensorOptions().dtype(torch::kUInt8).device(torch::kCPU).pinned_memory(true));
  void *status_dev = nullptr;
  OT_CHECK_HIP(hipHostGetDevicePointer(&status_dev, status_host.data_ptr(), 0));
  HostWriteGuard status_ready(stream);  // after status_host: destroyed, i.e. waited for, before it
  {
    ScopedTimer timer("prepare", stream);
    OT_CHECK(ot_row_splits(
        p_T, p_U, p_targets, (int32_t)N, (int32_t)S, row_splits,
        reinterpret_cast<int32_t *>(static_cast<char *>(status_dev) + host_splits_off),
        static_cast<ot_batch_status *>(status_dev), stream));
  }
  status_ready.record();

  // Two-part schedule for large batches.  The lattice kernel is a chain of
  // T+U dependent steps on a handful of CUs; run on a second stream, the part of
  // the batch whose denominators are ready overlaps with the streaming kernels
  // of the other part:
  //   main:  lse[rows < h]  lse[rows >= h]        grad[part A]      grad[part B]
  //   side:                 lattice+coeff[A]      lattice+coeff[B]
  // h is a row count, part A = the utterances that end at or before row h.
  const bool overlap = overlap_enabled() && dtype == OT_DTYPE_F32 && !have_den && N >= 2 &&
                       rows * V >= kOverlapMinElements;
  const int64_t half = overlap ? rows / 2 : rows;
  EventGuard lse_a_done, lse_b_done;

  // The first streaming kernel only reads and guards every index it derives
  // from device data, so it can run while the host waits for the facts.
  const bool blank_ok = (0 <= blank && blank < V);
  if (blank_ok) {
    ScopedTimer timer(from_log_softmax ? "gather" : have_den ? "gather_given_den" : "lse_gather",
                      stream);
    if (have_den) {
      OT_CHECK(ot_log_probs_given_den(p_logits, dtype, den, p_targets, p_U, row_splits, (int32_t)N,
                                      (int32_t)S, rows, (int32_t)V, blank, lp, stream));
    } else if (dtype != OT_DTYPE_F32) {
      OT_CHECK(ot_log_probs_half(p_logits, dtype, p_targets, p_U, row_splits, (int32_t)N,
                                 (int32_t)S, rows, (int32_t)V, blank, from_log_softmax, den, lp,
                                 stream));
    } else {
      OT_CHECK(ot_log_probs_range(p_logits32, p_targets, p_U, row_splits, (int32_t)N, (int32_t)S,
                                  rows, (int32_t)V, blank, from_log_softmax, 0, half, den, lp,
                                  stream));
    }
    if (overlap) {
      OT_CHECK_HIP(hipEventRecord(lse_a_done.ev, stream));
      OT_CHECK(ot_log_probs_range(p_logits32, p_targets, p_U, row_splits, (int32_t)N, (int32_t)S,
                                  rows, (int32_t)V, blank, from_log_softmax, half, rows, den, lp,
                                  stream));
      OT_CHECK_HIP(hipEventRecord(lse_b_done.ev, stream));
    }
  }
  // The lattice kernel goes out before the host wait as well: it writes workspace
  // only and checks on the device what its memory safety rests on, with
  // targets.size(1) + 1 columns (what target_lengths.max() + 1 must be, checked below).
  // The host's wake-up and its remaining launches then hide behind it even when the
  // first kernel is the short gather of log-softmax input.
  torch::Tensor scores = torch::empty({N}, logits.options().dtype(torch::kFloat));
  const bool early_lattice = blank_ok && !overlap;
  if (early_lattice) {
    ScopedTimer timer("alpha_beta", stream);
    OT_CHECK(ot_alpha_beta_guarded(lp, p_T, p_U, row_splits, (int32_t)N, (int32_t)S + 1,
                                   one_sym_per_frame, rows, alpha, beta, scores.data_ptr<float>(),
                                   scores_beta, stream));
  }
  status_ready.wait();
  const ot_batch_status st = *reinterpret_cast<const ot_batch_status *>(status_host.data_ptr());
  const int32_t *splits_host = reinterpret_cast<const int32_t *>(
      static_cast<const char *>(status_host.data_ptr()) + host_splits_off);

  check_batch_values(logits, targets, st.sum_tu, S > 0 ? (int64_t)st.targets_max : INT32_MIN,
                     st.target_len_max, blank);
  // beyond the reference (which has undefined behaviour for these): a negative id among the
  // entries that are read, u < target_lengths[b]; padding behind them is never read
  // (kernels.cu:49-50) and may hold anything below logits.size(1), e.g. -1
  TORCH_CHECK(S == 0 || st.targets_min >= 0, "targets.min() over the valid entries is ",
              st.targets_min, ". Expect targets >= 0");
  TORCH_CHECK(st.logit_len_min >= 1 && st.target_len_min >= 0,
              "Expect logit_lengths >= 1 and target_lengths >= 0, but the minima are ",
              st.logit_len_min, " and ", st.target_len_min);
  const int32_t max_u1 = st.target_len_max + 1;
  // the lattice kernel addresses one utterance's cells with 32-bit byte offsets
  TORCH_CHECK(((int64_t)st.logit_len_max + 1300) * max_u1 < ((int64_t)1 << 28),
              "an utterance with T = ", st.logit_len_max, " and up to ", max_u1,
              " lattice columns is too large for the lattice kernel");

  torch::Tensor gradient;
  const bool want_grad = logits.requires_grad();
  if (want_grad && !defer) {
    // cpu.cc:803 / cuda.cu:444: new tensor for log-softmax input;
    // cpu.cc:814 / cuda.cu:449: the logits buffer itself otherwise.
    gradient = from_log_softmax ? torch::empty_like(logits) : logits;
  }
  void *p_grad = gradient.defined() ? gradient.data_ptr() : nullptr;
  float *p_loss = nullptr;
  bool loss_done = false;
  if (reduced_loss) {
    *reduced_loss = torch::empty({}, logits.options().dtype(torch::kFloat));
    p_loss = reduced_loss->data_ptr<float>();
  }

  // lattice + per-row coefficients of utterances [b0, b1) on stream `s`
  auto lattice_part = [&](int32_t b0, int32_t b1, hipStream_t s) {
    if (!early_lattice) {
      ScopedTimer timer("alpha_beta", s);
      OT_CHECK(ot_alpha_beta_range(lp, p_T, p_U, row_splits, (int32_t)N, max_u1,
                                   one_sym_per_frame, b0, b1, alpha, beta,
                                   scores.data_ptr<float>(), scores_beta, s));
    }
    if (want_grad && p_loss && !loss_done && b0 == 0 && b1 == N) {
      ScopedTimer timer("row_coeff", s);
      OT_CHECK(ot_row_coefficients_loss(lp, den, alpha, beta, p_targets, p_T, p_U, row_splits,
                                        (int32_t)N, (int32_t)S, rows, blank, from_log_softmax,
                                        one_sym_per_frame, (float)grad_scale, coef,
                                        scores.data_ptr<float>(), (float)grad_scale, p_loss, s));
      loss_done = true;
    } else if (want_grad) {
      ScopedTimer timer("row_coeff", s);
      OT_CHECK(ot_row_coefficients_range(lp, den, alpha, beta, p_targets, p_T, p_U, row_splits,
                                         (int32_t)N, (int32_t)S, rows, blank, from_log_softmax,
                                         one_sym_per_frame, (float)grad_scale, splits_host[b0],
                                         splits_host[b1], coef, s));
    }
  };
  auto gradient_part = [&](int32_t b0, int32_t b1) {
    if (!p_grad) return;
    ScopedTimer timer(from_log_softmax ? "grad_logsoftmax" : "grad_logits", stream);
    if (dtype != OT_DTYPE_F32) {
      OT_CHECK(ot_gradient_apply_half(p_logits, dtype, coef, rows, (int32_t)V, from_log_softmax,
                                      (float)grad_scale, nullptr, p_grad, stream));
      return;
    }
    OT_CHECK(ot_gradient_apply_range(p_logits32, coef, rows, (int32_t)V, from_log_softmax,
                                     (float)grad_scale, splits_host[b0], splits_host[b1],
                                     static_cast<float *>(p_grad), stream));
  };

  // part A = utterances that lie completely in rows [0, half)
  int32_t b_split = 0;
  if (overlap) {
    while (b_split < N && (int64_t)splits_host[b_split + 1] <= half) ++b_split;
  }
  if (overlap && b_split >= 1 && b_split < N) {
    hipStream_t side =
        c10::hip::getStreamFromPoolMasqueradingAsCUDA(false, logits.device().index()).stream();
    EventGuard part_a_done, part_b_done;
    OT_CHECK_HIP(hipStreamWaitEvent(side, lse_a_done.ev, 0));
    lattice_part(0, b_split, side);
    OT_CHECK_HIP(hipEventRecord(part_a_done.ev, side));
    OT_CHECK_HIP(hipStreamWaitEvent(side, lse_b_done.ev, 0));
    lattice_part(b_split, (int32_t)N, side);
    OT_CHECK_HIP(hipEventRecord(part_b_done.ev, side));
    // `scores`, the workspace and the gradient are next used on the main stream,
    // which waits for both parts here; nothing on the side stream outlives this call
    OT_CHECK_HIP(hipStreamWaitEvent(stream, part_a_done.ev, 0));
    gradient_part(0, b_split);
    OT_CHECK_HIP(hipStreamWaitEvent(stream, part_b_done.ev, 0));
    gradient_part(b_split, (int32_t)N);
  } else {
    lattice_part(0, (int32_t)N, stream);
    gradient_part(0, (int32_t)N);
  }
  if (p_loss && !loss_done) {
    ScopedTimer timer("negative_sum", stream);
    OT_CHECK(ot_negative_sum(scores.data_ptr<float>(), (int32_t)N, (float)grad_scale, p_loss,
                             stream));
  }
  if (gradient.defined()) return {scores, gradient};
  return {scores, torch::nullopt};
}

// Signature and keyword names of the reference binding
// (optimized_transducer.cc:14-18).
std::pair<torch::Tensor, torch::optional<torch::Tensor>> compute_transducer_loss(
    torch::Tensor &logits, const torch::Tensor &targets, const torch::Tensor &logit_lengths,
    const torch::Tensor &target_lengths, int32_t blank, bool from_log_softmax,
    bool one_sym_per_frame) {
  return compute_impl(logits, targets, logit_lengths, target_lengths, blank, from_log_softmax,
                      one_sym_per_frame, 1.0, nullptr);
}

std::pair<torch::Tensor, torch::optional<torch::Tensor>> compute_transducer_loss_scaled(
    torch::Tensor &logits, const torch::Tensor &targets, const torch::Tensor &logit_lengths,
    const torch::Tensor &target_lengths, int32_t blank, bool from_log_softmax,
    bool one_sym_per_frame, double grad_scale,
    const torch::optional<torch::Tensor> &denominators) {
  return compute_impl(logits, targets, logit_lengths, target_lengths, blank, from_log_softmax,
                      one_sym_per_frame, grad_scale, nullptr, denominators);
}

// Forward half of the deferred mode: everything but the (rows, V) pass.  Returns
// (scores, per-row coefficients); the coefficients are None when logits does not
// require grad.  Nothing is written to logits.
std::pair<torch::Tensor, torch::optional<torch::Tensor>> compute_transducer_loss_deferred(
    torch::Tensor &logits, const torch::Tensor &targets, const torch::Tensor &logit_lengths,
    const torch::Tensor &target_lengths, int32_t blank, bool from_log_softmax,
    bool one_sym_per_frame, double grad_scale,
    const torch::optional<torch::Tensor> &denominators) {
  torch::Tensor coefficients;
  auto out = compute_impl(logits, targets, logit_lengths, target_lengths, blank, from_log_softmax,
                          one_sym_per_frame, grad_scale, &coefficients, denominators);
  if (coefficients.defined()) return {out.first, coefficients};
  return {out.first, torch::nullopt};
}

// compute_transducer_loss_scaled / _deferred that also return the reduced loss
// -grad_scale * scores.sum() (transducer_loss.py:145-147 with grad_scale = 1 for
// "sum" and 1/N for "mean"): (scores, gradient or coefficients or None, loss).
std::tuple<torch::Tensor, torch::optional<torch::Tensor>, torch::Tensor>
compute_transducer_loss_reduced(torch::Tensor &logits, const torch::Tensor &targets,
                                const torch::Tensor &logit_lengths,
                                const torch::Tensor &target_lengths, int32_t blank,
                                bool from_log_softmax, bool one_sym_per_frame, double grad_scale,
                                const torch::optional<torch::Tensor> &denominators) {
  torch::Tensor loss;
  auto out = compute_impl(logits, targets, logit_lengths, target_lengths, blank, from_log_softmax,
                          one_sym_per_frame, grad_scale, nullptr, denominators, &loss);
  return {out.first, out.second, loss};
}

std::tuple<torch::Tensor, torch::optional<torch::Tensor>, torch::Tensor>
compute_transducer_loss_deferred_reduced(torch::Tensor &logits, const torch::Tensor &targets,
                                         const torch::Tensor &logit_lengths,
                                         const torch::Tensor &target_lengths, int32_t blank,
                                         bool from_log_softmax, bool one_sym_per_frame,
                                         double grad_scale,
                                         const torch::optional<torch::Tensor> &denominators) {
  torch::Tensor coefficients, loss;
  auto out = compute_impl(logits, targets, logit_lengths, target_lengths, blank, from_log_softmax,
                          one_sym_per_frame, grad_scale, &coefficients, denominators, &loss);
  if (coefficients.defined()) return {out.first, coefficients, loss};
  return {out.first, torch::nullopt, loss};
}

// Backward half: the one pass over (rows, V), with loss_grad (a one-element float
// tensor on the device) folded in.  Logits input: `logits` is overwritten and
// returned (cuda.cu:449); log-softmax input: a new tensor (cuda.cu:444).
torch::Tensor apply_deferred_gradient(torch::Tensor &logits, const torch::Tensor &coefficients,
                                      bool from_log_softmax, double grad_scale,
                                      const torch::Tensor &loss_grad) {
  const int dtype = half_dtype(logits);
  TORCH_CHECK(logits.is_cuda() && (dtype != OT_DTYPE_F32 || logits.scalar_type() == torch::kFloat) &&
                  logits.dim() == 2 && logits.is_contiguous(),
              "apply_deferred_gradient: logits must be a contiguous 2-D float32, float16 or "
              "bfloat16 HIP tensor");
  const int64_t rows = logits.size(0), V = logits.size(1);
  TORCH_CHECK(rows > 0 && V > 0 && rows <= INT32_MAX && V <= INT32_MAX,
              "apply_deferred_gradient: bad logits shape");
  TORCH_CHECK(coefficients.is_cuda() && coefficients.device() == logits.device() &&
                  coefficients.scalar_type() == torch::kUInt8 && coefficients.is_contiguous() &&
                  coefficients.numel() == (int64_t)ot_gradient_scratch_bytes(rows),
              "apply_deferred_gradient: coefficients do not belong to these logits");
  TORCH_CHECK(loss_grad.is_cuda() && loss_grad.device() == logits.device() &&
                  loss_grad.scalar_type() == torch::kFloat && loss_grad.numel() == 1,
              "apply_deferred_gradient: loss_grad must be one float32 on the device of logits");
  c10::hip::HIPGuardMasqueradingAsCUDA device_guard(logits.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  torch::Tensor gradient = from_log_softmax ? torch::empty_like(logits) : logits;
  ScopedTimer timer(from_log_softmax ? "grad_logsoftmax" : "grad_logits", stream);
  if (dtype != OT_DTYPE_F32) {
    OT_CHECK(ot_gradient_apply_half(logits.data_ptr(), dtype, coefficients.data_ptr(), rows,
                                    (int32_t)V, from_log_softmax, (float)grad_scale,
                                    loss_grad.data_ptr<float>(), gradient.data_ptr(), stream));
    return gradient;
  }
  OT_CHECK(ot_gradient_apply_device_factor(logits.data_ptr<float>(), coefficients.data_ptr(), rows,
                                           (int32_t)V, from_log_softmax, (float)grad_scale,
                                           loss_grad.data_ptr<float>(),
                                           gradient.data_ptr<float>(), stream));
  return gradient;
}

// 0-dim loss = -scale * scores.sum() in one launch (replaces `-1 * scores` followed
// by .sum() / .mean(), transducer_loss.py:145-147).
torch::Tensor negative_sum(const torch::Tensor &scores, double scale) {
  TORCH_CHECK(scores.is_cuda() && scores.scalar_type() == torch::kFloat && scores.dim() == 1 &&
                  scores.is_contiguous() && scores.numel() > 0 && scores.numel() <= INT32_MAX,
              "negative_sum: scores must be a non-empty contiguous 1-D float32 HIP tensor");
  c10::hip::HIPGuardMasqueradingAsCUDA device_guard(scores.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  torch::Tensor loss = torch::empty({}, scores.options());
  ScopedTimer timer("negative_sum", stream);
  OT_CHECK(ot_negative_sum(scores.data_ptr<float>(), (int32_t)scores.numel(), (float)scale,
                           loss.data_ptr<float>(), stream));
  return loss;
}

// x *= loss_grad with loss_grad read on the device (no host synchronisation);
// the kernel returns immediately when loss_grad == 1.
void scale_by_device_scalar_(torch::Tensor &x, const torch::Tensor &factor) {
  TORCH_CHECK(x.is_cuda() && factor.is_cuda() && x.device() == factor.device(),
              "scale_by_device_scalar_: both tensors must be on the same HIP device");
  const int dtype = half_dtype(x);
  TORCH_CHECK((dtype != OT_DTYPE_F32 || x.scalar_type() == torch::kFloat) &&
                  factor.scalar_type() == torch::kFloat,
              "scale_by_device_scalar_: x must be float32, float16 or bfloat16 and factor float32");
  TORCH_CHECK(x.is_contiguous() && factor.numel() == 1,
              "scale_by_device_scalar_: x must be contiguous and factor a single element");
  c10::hip::HIPGuardMasqueradingAsCUDA device_guard(x.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  ScopedTimer timer("scale", stream);
  if (dtype != OT_DTYPE_F32) {
    OT_CHECK(ot_scale_by_device_scalar_half(x.data_ptr(), dtype, x.numel(),
                                            factor.data_ptr<float>(), stream));
    return;
  }
  OT_CHECK(ot_scale_by_device_scalar(x.data_ptr<float>(), x.numel(), factor.data_ptr<float>(),
                                     stream));
}

// ---- packed joiner input (the reference's README.md:166-177, done on the device) ----

int activation_code(const std::string &name) {
  if (name == "none") return OT_ACT_NONE;
  if (name == "tanh") return OT_ACT_TANH;
  if (name == "relu") return OT_ACT_RELU;
  TORCH_CHECK(false, "activation must be 'none', 'tanh' or 'relu', got '", name, "'");
  return -1;
}

void check_joiner_inputs(const torch::Tensor &enc, const torch::Tensor &dec,
                         const torch::Tensor &logit_lengths, const torch::Tensor &target_lengths) {
  TORCH_CHECK(enc.is_cuda() && dec.is_cuda() && logit_lengths.is_cuda() && target_lengths.is_cuda() &&
                  enc.device() == dec.device() && enc.device() == logit_lengths.device() &&
                  enc.device() == target_lengths.device(),
              "pack_joiner: all tensors must be on the same HIP device (this build has no CPU "
              "implementation)");
  TORCH_CHECK(enc.scalar_type() == torch::kFloat && dec.scalar_type() == torch::kFloat,
              "pack_joiner: encoder_out and decoder_out must be float32");
  TORCH_CHECK(logit_lengths.scalar_type() == torch::kInt32 &&
                  target_lengths.scalar_type() == torch::kInt32,
              "pack_joiner: logit_lengths and target_lengths must be int32");
  TORCH_CHECK(enc.dim() == 3 && dec.dim() == 3 && logit_lengths.dim() == 1 &&
                  target_lengths.dim() == 1,
              "pack_joiner: expected encoder_out (N, T, D), decoder_out (N, U+1, D) and 1-D lengths");
  TORCH_CHECK(enc.is_contiguous() && dec.is_contiguous() && logit_lengths.is_contiguous() &&
                  target_lengths.is_contiguous(),
              "pack_joiner: tensors must be contiguous");
  const int64_t N = enc.size(0);
  TORCH_CHECK(N > 0 && dec.size(0) == N && logit_lengths.size(0) == N && target_lengths.size(0) == N,
              "pack_joiner: batch sizes differ: ", enc.size(0), ", ", dec.size(0), ", ",
              logit_lengths.size(0), ", ", target_lengths.size(0));
  TORCH_CHECK(enc.size(2) == dec.size(2) && enc.size(2) > 0,
              "pack_joiner: encoder_out and decoder_out differ in the last dimension: ", enc.size(2),
              " vs ", dec.size(2));
  TORCH_CHECK(enc.size(1) > 0 && dec.size(1) > 0 && N * enc.size(1) <= INT32_MAX &&
                  N * dec.size(1) <= INT32_MAX && enc.size(2) <= INT32_MAX && N <= 65535,
              "pack_joiner: tensor sizes out of range");
}

// (packed (rows, D), row_splits (N+1) int32)
std::pair<torch::Tensor, torch::Tensor> joiner_pack(
    const torch::Tensor &enc, const torch::Tensor &dec, const torch::Tensor &logit_lengths,
    const torch::Tensor &target_lengths, const std::string &activation,
    const std::string &out_dtype) {
  const int act = activation_code(activation);
  check_joiner_inputs(enc, dec, logit_lengths, target_lengths);
  const int64_t N = enc.size(0), Tmax = enc.size(1), U1max = dec.size(1), D = enc.size(2);
  const int odt = out_dtype == "float16" ? OT_DTYPE_F16 : out_dtype == "bfloat16" ? OT_DTYPE_BF16 : OT_DTYPE_F32;
  TORCH_CHECK(odt != OT_DTYPE_F32 || out_dtype == "float32",
              "pack_joiner: out_dtype must be float32, float16 or bfloat16, got ", out_dtype);
  TORCH_CHECK(odt == OT_DTYPE_F32 || D % 8 == 0,
              "pack_joiner: a 16-bit output needs D to be a multiple of 8, got ", D);
  c10::hip::HIPGuardMasqueradingAsCUDA device_guard(enc.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();

  torch::Tensor row_splits = torch::empty({N + 1}, logit_lengths.options());
  torch::Tensor status_host = torch::empty(
      {(int64_t)sizeof(ot_batch_status)},
      torch::TensorOptions().dtype(torch::kUInt8).device(torch::kCPU).pinned_memory(true));
  void *status_dev = nullptr;
  OT_CHECK_HIP(hipHostGetDevicePointer(&status_dev, status_host.data_ptr(), 0));
  HostWriteGuard ready(stream);
  {
    ScopedTimer timer("prepare", stream);
    OT_CHECK(ot_row_splits(logit_lengths.data_ptr<int32_t>(), target_lengths.data_ptr<int32_t>(),
                           nullptr, (int32_t)N, 0, row_splits.data_ptr<int32_t>(), nullptr,
                           static_cast<ot_batch_status *>(status_dev), stream));
  }
  ready.record();
  ready.wait();  // the output's size is a batch fact
  const ot_batch_status st = *reinterpret_cast<const ot_batch_status *>(status_host.data_ptr());
  TORCH_CHECK(st.logit_len_min >= 1 && st.target_len_min >= 0,
              "pack_joiner: expect logit_lengths >= 1 and target_lengths >= 0, but the minima are ",
              st.logit_len_min, " and ", st.target_len_min);
  TORCH_CHECK(st.logit_len_max <= Tmax, "pack_joiner: logit_lengths.max() is ", st.logit_len_max,
              " but encoder_out has ", Tmax, " frames");
  TORCH_CHECK((int64_t)st.target_len_max + 1 <= U1max, "pack_joiner: target_lengths.max() + 1 is ",
              (int64_t)st.target_len_max + 1, " but decoder_out has ", U1max, " positions");
  const int64_t rows = st.sum_tu;
  TORCH_CHECK(rows > 0 && rows <= INT32_MAX, "pack_joiner: sum of T * (U + 1) is ", rows,
              ", outside (0, 2^31)");

  torch::Tensor out = torch::empty(
      {rows, D}, enc.options().dtype(odt == OT_DTYPE_F16    ? torch::kHalf
                                     : odt == OT_DTYPE_BF16 ? torch::kBFloat16
                                                            : torch::kFloat));
  {
    ScopedTimer timer("joiner_pack", stream);
    if (odt == OT_DTYPE_F32) {
      OT_CHECK(ot_joiner_pack(enc.data_ptr<float>(), dec.data_ptr<float>(),
                              logit_lengths.data_ptr<int32_t>(), target_lengths.data_ptr<int32_t>(),
                              row_splits.data_ptr<int32_t>(), (int32_t)N, (int32_t)Tmax,
                              (int32_t)U1max, (int32_t)D, act, out.data_ptr<float>(), stream));
    } else {
      OT_CHECK(ot_joiner_pack_half(enc.data_ptr<float>(), dec.data_ptr<float>(),
                                   logit_lengths.data_ptr<int32_t>(),
                                   target_lengths.data_ptr<int32_t>(), row_splits.data_ptr<int32_t>(),
                                   (int32_t)N, (int32_t)Tmax, (int32_t)U1max, (int32_t)D, act, odt,
                                   out.data_ptr(), stream));
    }
  }
  return {out, row_splits};
}

// (grad_encoder_out (N, T, D), grad_decoder_out (N, U+1, D)) for grad_out (rows, D)
std::pair<torch::Tensor, torch::Tensor> joiner_unpack_grad(
    const torch::Tensor &grad_out, const torch::Tensor &enc, const torch::Tensor &dec,
    const torch::Tensor &logit_lengths, const torch::Tensor &target_lengths,
    const torch::Tensor &row_splits, const std::string &activation) {
  const int act = activation_code(activation);
  check_joiner_inputs(enc, dec, logit_lengths, target_lengths);
  const int64_t N = enc.size(0), Tmax = enc.size(1), U1max = dec.size(1), D = enc.size(2);
  TORCH_CHECK(grad_out.is_cuda() && grad_out.device() == enc.device() &&
                  (grad_out.scalar_type() == torch::kFloat || half_dtype(grad_out) != OT_DTYPE_F32) &&
                  grad_out.dim() == 2 && grad_out.size(1) == D && grad_out.is_contiguous(),
              "pack_joiner backward: the gradient must be a contiguous float32, float16 or bfloat16 (rows, ", D,
              ") tensor on the device of encoder_out");
  TORCH_CHECK(row_splits.is_cuda() && row_splits.device() == enc.device() &&
                  row_splits.scalar_type() == torch::kInt32 && row_splits.dim() == 1 &&
                  row_splits.size(0) == N + 1 && row_splits.is_contiguous(),
              "pack_joiner backward: row_splits must be the (N+1,) int32 tensor of the forward call");
  c10::hip::HIPGuardMasqueradingAsCUDA device_guard(enc.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  const size_t ws_bytes =
      ot_joiner_unpack_workspace_bytes((int32_t)N, (int32_t)Tmax, (int32_t)U1max, (int32_t)D);
  torch::Tensor workspace = torch::empty({(int64_t)ws_bytes}, enc.options().dtype(torch::kUInt8));
  torch::Tensor grad_enc = torch::empty_like(enc);
  torch::Tensor grad_dec = torch::empty_like(dec);
  ScopedTimer timer("joiner_unpack_grad", stream);
  OT_CHECK(ot_joiner_unpack_grad_from(grad_out.data_ptr(), half_dtype(grad_out), enc.data_ptr<float>(),
                                 dec.data_ptr<float>(), logit_lengths.data_ptr<int32_t>(),
                                 target_lengths.data_ptr<int32_t>(), row_splits.data_ptr<int32_t>(),
                                 (int32_t)N, (int32_t)Tmax, (int32_t)U1max, (int32_t)D, act,
                                 workspace.data_ptr(), ws_bytes, grad_enc.data_ptr<float>(),
                                 grad_dec.data_ptr<float>(), stream));
  return {grad_enc, grad_dec};
}

}  // namespace

// Output projection of the joiner with the denominators of the loss from the
// accumulators (ot_joiner_project): logits (rows, V) float32 or of x's dtype, den (rows).
std::pair<torch::Tensor, torch::Tensor> joiner_project(const torch::Tensor &x,
                                                       const torch::Tensor &weight,
                                                       const torch::optional<torch::Tensor> &bias,
                                                       bool float32_logits) {
  const int dtype = half_dtype(x);
  TORCH_CHECK(dtype != OT_DTYPE_F32, "joiner_project takes float16 or bfloat16 x, got ", x.scalar_type());
  TORCH_CHECK(x.is_cuda() && weight.device() == x.device(), "x and weight must be on one HIP device");
  TORCH_CHECK(x.dim() == 2 && weight.dim() == 2 && x.size(1) == weight.size(1) &&
                  weight.scalar_type() == x.scalar_type() && x.is_contiguous() && weight.is_contiguous(),
              "expect contiguous x (rows, D) and weight (V, D) of one dtype");
  const int64_t rows = x.size(0), D = x.size(1), V = weight.size(0);
  TORCH_CHECK(rows > 0 && V > 0 && D > 0 && D % 64 == 0 && rows <= INT32_MAX,
              "joiner_project needs rows > 0, V > 0 and D a positive multiple of 64, got rows = ", rows,
              ", V = ", V, ", D = ", D);
  torch::Tensor b;
  if (bias.has_value() && bias->defined()) {
    TORCH_CHECK(bias->dim() == 1 && bias->size(0) == V && bias->device() == x.device(),
                "bias must have shape (V,) on the device of x");
    b = bias->to(torch::kFloat).contiguous();
  }
  c10::hip::HIPGuardMasqueradingAsCUDA device_guard(x.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  torch::Tensor logits =
      torch::empty({rows, V}, x.options().dtype(float32_logits ? torch::kFloat : x.scalar_type()));
  torch::Tensor den = torch::empty({rows}, x.options().dtype(torch::kFloat));
  // room for one partial log-sum-exp per row and 256-column pass: with it the passes of a
  // block of rows run side by side on one XCD and x is read from HBM once
  const size_t ws_bytes = ot_joiner_project_workspace_bytes(rows, (int32_t)V);
  torch::Tensor workspace;
  if (ws_bytes > 0) workspace = torch::empty({(int64_t)ws_bytes}, x.options().dtype(torch::kUInt8));
  {
    ScopedTimer timer("joiner_project", stream);
    OT_CHECK(ot_joiner_project_ws(x.data_ptr(), weight.data_ptr(),
                                  b.defined() ? b.data_ptr<float>() : nullptr, dtype, rows, (int32_t)D,
                                  (int32_t)V, logits.data_ptr(), float32_logits ? OT_DTYPE_F32 : dtype,
                                  den.data_ptr<float>(), ws_bytes > 0 ? workspace.data_ptr() : nullptr,
                                  ws_bytes, stream));
  }
  return {logits, den};
}

// Gradient of that projection with respect to weight and bias (ot_joiner_weight_grad):
// (grad_weight (V, D) of x's dtype, grad_bias (V) float32) from the gradient of the logits.
std::pair<torch::Tensor, torch::Tensor> joiner_weight_grad(const torch::Tensor &grad_logits,
                                                           const torch::Tensor &x) {
  const int dtype = half_dtype(x);
  TORCH_CHECK(dtype != OT_DTYPE_F32, "joiner_weight_grad takes float16 or bfloat16 x, got ", x.scalar_type());
  TORCH_CHECK(x.is_cuda() && grad_logits.device() == x.device(), "grad_logits and x must be on one HIP device");
  TORCH_CHECK(x.dim() == 2 && grad_logits.dim() == 2 && x.size(0) == grad_logits.size(0) &&
                  grad_logits.scalar_type() == x.scalar_type() && x.is_contiguous() &&
                  grad_logits.is_contiguous(),
              "expect contiguous grad_logits (rows, V) and x (rows, D) of one dtype");
  const int64_t rows = x.size(0), D = x.size(1), V = grad_logits.size(1);
  TORCH_CHECK(rows > 0 && rows <= INT32_MAX && V > 0 && D > 0 && V % 8 == 0 && D % 8 == 0,
              "joiner_weight_grad needs rows > 0 and V, D positive multiples of 8, got rows = ", rows,
              ", V = ", V, ", D = ", D);
  c10::hip::HIPGuardMasqueradingAsCUDA device_guard(x.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  const size_t ws_bytes = ot_joiner_weight_grad_workspace_bytes(rows, (int32_t)V, (int32_t)D);
  torch::Tensor workspace = torch::empty({(int64_t)ws_bytes}, x.options().dtype(torch::kUInt8));
  torch::Tensor grad_w = torch::empty({V, D}, x.options());
  torch::Tensor grad_b = torch::empty({V}, x.options().dtype(torch::kFloat));
  {
    ScopedTimer timer("joiner_weight_grad", stream);
    OT_CHECK(ot_joiner_weight_grad(grad_logits.data_ptr(), x.data_ptr(), dtype, rows, (int32_t)V,
                                   (int32_t)D, workspace.data_ptr(), ws_bytes, grad_w.data_ptr(),
                                   grad_b.data_ptr<float>(), stream));
  }
  return {grad_w, grad_b};
}

PYBIND11_MODULE(_optimized_transducer, m) {
  m.doc() = "MI355X-native transducer loss (drop-in for optimized_transducer's extension module)";
#ifdef OT_BUILT_WITH_TORCH
  // the reference records the same fact in a generated torch_version.py
  // (optimized_transducer/python/optimized_transducer/__init__.py:3-9)
  m.attr("built_with_torch") = OT_BUILT_WITH_TORCH;
#endif
  m.def("compute_transducer_loss", &compute_transducer_loss, py::arg("logits"),
        py::arg("targets"), py::arg("logit_lengths"), py::arg("target_lengths"),
        py::arg("blank"), py::arg("from_log_softmax"), py::arg("one_sym_per_frame"));
  m.def("compute_transducer_loss_scaled", &compute_transducer_loss_scaled, py::arg("logits"), py::arg("targets"),
        py::arg("logit_lengths"), py::arg("target_lengths"), py::arg("blank"),
        py::arg("from_log_softmax"), py::arg("one_sym_per_frame"), py::arg("grad_scale"),
        py::arg("denominators") = py::none(),
        "Same as compute_transducer_loss with the gradient multiplied by grad_scale in the "
        "gradient kernel (folds the `grad /= N` of reduction='mean'); denominators: the per-row "
        "log-sum-exp of the logits if already known (joiner_project), else None.");
  m.def("compute_transducer_loss_deferred", &compute_transducer_loss_deferred, py::arg("logits"),
        py::arg("targets"), py::arg("logit_lengths"), py::arg("target_lengths"), py::arg("blank"),
        py::arg("from_log_softmax"), py::arg("one_sym_per_frame"), py::arg("grad_scale"),
        py::arg("denominators") = py::none(),
        "Everything but the (rows, V) gradient pass: returns (scores, per-row coefficients or "
        "None) and leaves logits untouched.");
  m.def("compute_transducer_loss_reduced", &compute_transducer_loss_reduced, py::arg("logits"),
        py::arg("targets"), py::arg("logit_lengths"), py::arg("target_lengths"), py::arg("blank"),
        py::arg("from_log_softmax"), py::arg("one_sym_per_frame"), py::arg("grad_scale"),
        py::arg("denominators") = py::none(),
        "compute_transducer_loss_scaled that also returns the 0-dim loss "
        "-grad_scale * scores.sum(): (scores, grad or None, loss).");
  m.def("compute_transducer_loss_deferred_reduced", &compute_transducer_loss_deferred_reduced,
        py::arg("logits"), py::arg("targets"), py::arg("logit_lengths"),
        py::arg("target_lengths"), py::arg("blank"), py::arg("from_log_softmax"),
        py::arg("one_sym_per_frame"), py::arg("grad_scale"), py::arg("denominators") = py::none(),
        "compute_transducer_loss_deferred that also returns the 0-dim loss: "
        "(scores, coefficients or None, loss).");
  m.def("apply_deferred_gradient", &apply_deferred_gradient, py::arg("logits"),
        py::arg("coefficients"), py::arg("from_log_softmax"), py::arg("grad_scale"),
        py::arg("loss_grad"),
        "The (rows, V) gradient pass for the coefficients of compute_transducer_loss_deferred, "
        "times grad_scale and the device scalar loss_grad.");
  m.def("negative_sum", &negative_sum, py::arg("scores"), py::arg("scale"),
        "0-dim tensor -scale * scores.sum(), one launch.");
  m.def("scale_by_device_scalar_", &scale_by_device_scalar_, py::arg("x"), py::arg("factor"));
  m.def("joiner_pack", &joiner_pack, py::arg("encoder_out"), py::arg("decoder_out"),
        py::arg("logit_lengths"), py::arg("target_lengths"), py::arg("activation"),
        py::arg("out_dtype") = "float32",
        "Packed joiner input act(enc[b,t] + dec[b,u]) for the valid (t, u) cells, in the row order "
        "of the loss; returns (packed (rows, D), row_splits).");
  m.def("joiner_unpack_grad", &joiner_unpack_grad, py::arg("grad_out"), py::arg("encoder_out"),
        py::arg("decoder_out"), py::arg("logit_lengths"), py::arg("target_lengths"),
        py::arg("row_splits"), py::arg("activation"),
        "Gradient of joiner_pack: (grad_encoder_out, grad_decoder_out).");
  m.def("joiner_project", &joiner_project, py::arg("x"), py::arg("weight"), py::arg("bias"),
        py::arg("float32_logits"),
        "logits = x @ weight.T + bias for float16 / bfloat16 x (rows, D) and weight (V, D) on the "
        "matrix cores, and their per-row log-sum-exp: returns (logits, denominators).");
  m.def("joiner_weight_grad", &joiner_weight_grad, py::arg("grad_logits"), py::arg("x"),
        "Backward of joiner_project in its parameters: (grad_logits.T @ x in x's dtype, "
        "grad_logits.sum(0) in float32) for float16 / bfloat16 operands, float32 accumulation.");
  m.def("set_profiling", &set_profiling, py::arg("on"));
  m.def("set_overlap", &set_overlap, py::arg("on"),
        "Run the lattice kernel of one half of a large batch on a second stream while the "
        "streaming kernels of the other half run (off by default).");
  m.def("take_profile", &take_profile);
}
