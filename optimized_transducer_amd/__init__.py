"""MI355X-native transducer (RNN-T) loss: a drop-in for ``optimized_transducer``.

Same entry points as the reference package
(optimized_transducer/python/optimized_transducer/__init__.py:11):
``transducer_loss`` and ``TransducerLoss``.  All computation happens in
hand-written gfx950 HIP kernels; there is no CPU implementation, and without
the in-tree extension (``python -m optimized_transducer_amd.build``) every name
of this package raises ``ImportError``.
"""
try:
    from . import _optimized_transducer  # noqa: F401
    _load_error = None
except ImportError as e:  # an unbuilt tree
    _load_error = e

if _load_error is None:
    import torch as _torch

    # same guard as the reference package (optimized_transducer/__init__.py:5-9)
    _built = getattr(_optimized_transducer, "built_with_torch", _torch.__version__)
    if _torch.__version__.split("+")[0] != _built.split("+")[0]:
        raise ImportError(
            f"optimized_transducer_amd was built using PyTorch {_built}\n"
            f"But you are using PyTorch {_torch.__version__} to run it"
        )

    from .transducer_loss import TransducerLoss, TransducerLossFunction, transducer_loss  # noqa: E402,F401
    from .joiner import (PackJoinerFunction, ProjectJoinerFunction, joiner_transducer_loss,  # noqa: E402,F401
                         pack_joiner, project_joiner)
else:
    # Nothing works without the extension, and nothing pretends to: every name of the
    # package raises.  The import of the bare package itself succeeds so that
    # `python -m optimized_transducer_amd.build` can run in an unbuilt tree.
    class ExtensionNotBuilt(ImportError, AttributeError):
        """ImportError for `from optimized_transducer_amd import x`; also an AttributeError,
        so that hasattr(), getattr(..., default) and the import system's probes for
        submodules and dunder names behave as for any missing attribute."""

    def __getattr__(name):
        if name.startswith("__") and name.endswith("__"):
            raise AttributeError(name)
        raise ExtensionNotBuilt(
            "optimized_transducer_amd: the HIP extension is not built or failed to load (%s). "
            "Run `python -m optimized_transducer_amd.build` in the repository root." % (_load_error,)
        ) from _load_error

__all__ = ["TransducerLoss", "TransducerLossFunction", "transducer_loss", "PackJoinerFunction",
           "pack_joiner", "ProjectJoinerFunction", "project_joiner", "joiner_transducer_loss"]
