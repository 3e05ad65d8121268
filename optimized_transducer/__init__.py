"""``import optimized_transducer`` for code written against the reference package
(optimized_transducer/python/optimized_transducer/__init__.py:11 exports
``TransducerLoss`` and ``transducer_loss``): the same names, computed by the
MI355X implementation in ``optimized_transducer_amd``.  Put the repository root
on ``sys.path`` (or install it) and the import line of existing code need not
change.  Importing fails, like ``optimized_transducer_amd`` itself, when the HIP
extension has not been built.
"""
# through the submodule, as the reference does, so that the function and not the
# submodule ends up under the name `transducer_loss` (fails here when the HIP extension
# is not built)
from .transducer_loss import TransducerLoss, TransducerLossFunction, transducer_loss  # noqa: F401,E402
# what this build has beyond the reference, under the same roof
from optimized_transducer_amd import joiner_transducer_loss, pack_joiner, project_joiner  # noqa: F401,E402

__all__ = ["TransducerLoss", "transducer_loss", "pack_joiner", "project_joiner",
           "joiner_transducer_loss"]
