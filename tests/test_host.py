"""Host-side logic that needs no GPU: the C ABI surface, the drop-in Python
surface, and the argument checks (which mirror
optimized_transducer/csrc/transducer-loss.cc:33-66 and are compared message by
message with the compiled reference where oracle/_ref has been built)."""
import ctypes
import inspect
import os
import re
import subprocess
import sys

import pytest
import torch

import cabi
from oracle import ref_loader

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ----------------------------------------------------------------- C ABI
def declared_symbols():
    text = open(cabi.HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ot_[a-z_]+)\s*\(", text)))


def test_library_exports_every_symbol_the_header_declares():
    names = declared_symbols()
    assert {"ot_row_splits", "ot_log_probs", "ot_alpha_beta", "ot_gradient",
            "ot_transducer_loss"} <= set(names)
    lib = ctypes.CDLL(cabi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n


def test_header_is_plain_c_and_a_c_program_links_against_the_library(tmp_path):
    # the boundary is a C ABI: a C99 translation unit that includes the header and calls an
    # entry point which needs no device must compile with gcc, link and run
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_abi.c"
    src.write_text(
        '#include <stdio.h>\n#include "ot_transducer.h"\n'
        "int main(void) {\n"
        "  ot_batch_status s; (void)s;\n"
        "  if (sizeof(ot_batch_status) != 32) return 2;\n"
        "  if (ot_workspace_bytes(0, 10) != 0) return 3;\n"
        "  if (ot_transducer_loss_static(0, 0, 0, 0, 0, 1, 0, 1, 4, 0, 0, 0, 1.0f, 0, 0, 0, 0) >= 0) return 4;\n"
        '  printf("%s\\n", ot_error_string(OT_E_TOO_LARGE));\n'
        "  return 0;\n}\n")
    exe = tmp_path / "use_abi"
    libdir = os.path.dirname(cabi.LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I",
                    os.path.dirname(cabi.HEADER), str(src), "-o", str(exe), "-L", libdir,
                    "-l:" + os.path.basename(cabi.LIB_PATH), "-Wl,-rpath," + libdir], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert "OT_STATIC_WORKSPACE_BYTES" in out or "static" in out.lower(), out


def test_c_abi_rejects_bad_arguments_before_touching_the_device():
    L = cabi.lib()
    null = ctypes.c_void_p(0)
    i32, i64 = ctypes.c_int32, ctypes.c_int64
    assert L.ot_row_splits(null, null, null, i32(4), i32(3), null, null, null, null) == -1
    assert L.ot_row_ids(null, i32(1), i64(5), null, null) == -1
    assert L.ot_log_probs(null, null, null, null, i32(1), i32(0), i64(4), i32(8), i32(0), i32(0),
                          null, null, null) == -1
    one = ctypes.c_void_p(16)  # never dereferenced: the size checks fail first
    assert L.ot_alpha_beta(one, one, one, one, i32(1), i32((1 << 18) + 1), i32(0), one, one, one,
                           one, null) == -2  # OT_E_TOO_LONG
    assert L.ot_log_probs(one, one, one, one, i32(1), i32(1), i64(4), i32(8), i32(9), i32(0), one,
                          one, null) == -1  # blank >= V
    assert L.ot_gradient(null, null, null, null, null, null, null, null, null, i32(1), i32(0),
                         i64(1), i32(4), i32(0), i32(0), i32(0), ctypes.c_float(1), null, null,
                         null) == -1
    assert L.ot_workspace_bytes(i32(0), i64(10)) == 0
    n1 = L.ot_workspace_bytes(i32(4), i64(1000))
    n2 = L.ot_workspace_bytes(i32(4), i64(2000))
    assert 1000 * 44 <= n1 < n2 < 2000 * 44 + 4096 * 8
    assert L.ot_gradient_scratch_bytes(i64(10)) == 240
    assert b"OT_MAX_U1" in L.ot_error_string(-2)
    assert L.ot_error_string(0) == b"success"


# ------------------------------------------------------------ Python surface
def test_python_entry_points_keep_the_reference_signatures():
    import optimized_transducer_amd as ot
    # optimized_transducer/python/optimized_transducer/transducer_loss.py:312-321
    sig = inspect.signature(ot.transducer_loss)
    ref_names = ["logits", "targets", "logit_lengths", "target_lengths", "blank",
                 "from_log_softmax", "one_sym_per_frame", "reduction"]
    assert list(sig.parameters)[:8] == ref_names
    for extra in list(sig.parameters)[8:]:  # additions: keyword only, off by default
        assert sig.parameters[extra].kind is inspect.Parameter.KEYWORD_ONLY
        assert sig.parameters[extra].default in (False, None)
    assert sig.parameters["one_sym_per_frame"].default is False
    assert sig.parameters["reduction"].default == "mean"
    assert sig.parameters["from_log_softmax"].default is inspect.Parameter.empty
    # transducer_loss.py:174, :190-198
    init = inspect.signature(ot.TransducerLoss.__init__)
    assert list(init.parameters) == ["self", "blank", "reduction"]
    assert init.parameters["reduction"].default == "mean"
    fwd = inspect.signature(ot.TransducerLoss.forward)
    assert list(fwd.parameters) == ["self", "logits", "targets", "logit_lengths", "target_lengths",
                                    "from_log_softmax", "one_sym_per_frame"]
    assert fwd.parameters["one_sym_per_frame"].default is False
    m = ot.TransducerLoss(blank=0, reduction="sum")  # the reference's class cannot be called
    assert isinstance(m, torch.nn.Module) and m.blank == 0 and m.reduction == "sum"
    # optimized_transducer.cc:14-18: seven keyword-nameable arguments, no defaults
    doc = ot._optimized_transducer.compute_transducer_loss.__doc__
    for kw in ("logits", "targets", "logit_lengths", "target_lengths", "blank", "from_log_softmax",
               "one_sym_per_frame"):
        assert kw + ":" in doc


def _good():
    T = torch.tensor([3, 4], dtype=torch.int32)
    U = torch.tensor([2, 1], dtype=torch.int32)
    targets = torch.tensor([[1, 2], [2, 1]], dtype=torch.int32)
    logits = torch.randn(3 * 3 + 4 * 2, 5)
    return dict(logits=logits, targets=targets, logit_lengths=T, target_lengths=U, blank=0,
                from_log_softmax=False, one_sym_per_frame=False)


def _mutations():
    def m(**kw):
        a = _good()
        a.update(kw)
        return a
    g = _good()
    return {
        "logits dtype": m(logits=g["logits"].double()),
        "targets dtype": m(targets=g["targets"].long()),
        "logit_lengths dtype": m(logit_lengths=g["logit_lengths"].long()),
        "target_lengths dtype": m(target_lengths=g["target_lengths"].short()),
        "non contiguous": m(logits=torch.randn(5, 17).t()),
        "logits dim": m(logits=torch.randn(17 * 5)),
        "targets dim": m(targets=torch.tensor([1, 2], dtype=torch.int32)),
        "lengths size": m(logit_lengths=torch.tensor([3, 4, 5], dtype=torch.int32)),
        "sum_TU": m(logits=torch.randn(16, 5)),
        "targets max": m(targets=torch.tensor([[1, 5], [2, 1]], dtype=torch.int32)),
        "blank high": m(blank=5),
        "blank negative": m(blank=-1),
        "targets cols": m(targets=torch.tensor([[1, 2, 3], [2, 1, 1]], dtype=torch.int32)),
    }


def _message(fn, args):
    with pytest.raises(RuntimeError) as e:
        fn(**args)
    return str(e.value).split("\n")[0]


@pytest.mark.parametrize("name", sorted(_mutations()))
def test_argument_checks_raise_like_the_reference(name):
    import optimized_transducer_amd as ot
    args = _mutations()[name]
    msg = _message(ot._optimized_transducer.compute_transducer_loss, args)
    assert "no CPU implementation" not in msg, "bad argument went undetected: " + msg
    ref = ref_loader.load()
    if ref is not None:
        want = _message(ref.compute_transducer_loss, _mutations()[name])
        assert msg == want


@pytest.mark.skipif(torch.cuda.is_available(), reason="with a GPU, CPU tensors are computed on it")
def test_valid_cpu_tensors_fail_loudly_without_a_hip_device():
    # CPU tensors are staged through the GPU (tests/test_gpu_drop_in.py); without one there
    # is nothing to fall back to, and the call says so instead of computing on the host
    import optimized_transducer_amd as ot
    msg = _message(ot._optimized_transducer.compute_transducer_loss, _good())
    assert "no CPU implementation" in msg and "no HIP device" in msg
    with pytest.raises(RuntimeError, match="no HIP device"):
        ot.transducer_loss(**{k: v for k, v in _good().items()}, reduction="sum")


def test_the_reference_import_line_works():
    # optimized_transducer/python/optimized_transducer/__init__.py:11
    import optimized_transducer
    import optimized_transducer_amd as ot
    assert optimized_transducer.transducer_loss is ot.transducer_loss
    assert optimized_transducer.TransducerLoss is ot.TransducerLoss
    from optimized_transducer.transducer_loss import TransducerLossFunction
    assert TransducerLossFunction is ot.TransducerLossFunction
    # the additions are reachable under the same name
    for name in ("pack_joiner", "project_joiner", "joiner_transducer_loss"):
        assert getattr(optimized_transducer, name) is getattr(ot, name)


def test_reduction_none_is_rejected_like_the_reference():
    import optimized_transducer_amd as ot
    with pytest.raises(AssertionError):  # transducer_loss.py:133
        ot.transducer_loss(**_good(), reduction="none")


def test_product_never_imports_the_oracle():
    for root, _, files in os.walk(os.path.join(ROOT, "optimized_transducer_amd")):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(root, f)).read()
                assert "oracle" not in text.lower(), os.path.join(root, f)


def test_bench_refuses_more_than_one_gpu():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert p.returncode != 0 and "one GPU" in (p.stderr + p.stdout)
