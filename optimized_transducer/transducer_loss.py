"""Module path of the reference (optimized_transducer/python/optimized_transducer/
transducer_loss.py): ``from optimized_transducer.transducer_loss import ...``."""
from optimized_transducer_amd.transducer_loss import (TransducerLoss,  # noqa: F401
                                                      TransducerLossFunction, transducer_loss)
