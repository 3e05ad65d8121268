"""MI355X-native transducer (RNN-T) loss: a drop-in for ``optimized_transducer``.

Same entry points as the reference package
(optimized_transducer/python/optimized_transducer/__init__.py:11):
``transducer_loss`` and ``TransducerLoss``.  All computation happens in
hand-written gfx950 HIP kernels; there is no CPU implementation and importing
this package fails if the in-tree extension has not been built
(``python -m optimized_transducer_amd.build``).
"""
try:
    from . import _optimized_transducer  # noqa: F401
except ImportError as e:  # pragma: no cover - exercised only on an unbuilt tree
    raise ImportError(
        "optimized_transducer_amd: the HIP extension is not built or failed to load (%s). "
        "Run `python -m optimized_transducer_amd.build` in the repository root." % (e,)
    ) from e

import torch as _torch

# same guard as the reference package (optimized_transducer/__init__.py:5-9)
_built = getattr(_optimized_transducer, "built_with_torch", _torch.__version__)
if _torch.__version__.split("+")[0] != _built.split("+")[0]:
    raise ImportError(
        f"optimized_transducer_amd was built using PyTorch {_built}\n"
        f"But you are using PyTorch {_torch.__version__} to run it"
    )

from .transducer_loss import TransducerLoss, TransducerLossFunction, transducer_loss  # noqa: E402,F401
from .joiner import (PackJoinerFunction, ProjectJoinerFunction, pack_joiner,  # noqa: E402,F401
                     project_joiner)

__all__ = ["TransducerLoss", "TransducerLossFunction", "transducer_loss", "PackJoinerFunction",
           "pack_joiner", "ProjectJoinerFunction", "project_joiner"]
