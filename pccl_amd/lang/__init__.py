"""Python collective IR (the reference's ``pccl/lang``) and schedule emitters."""
from .graph import DirectedGraph  # noqa: F401
from .ir import Chunk, CollectiveIR, Device, DeviceType, Link, PrimitiveOp, PrimitiveOpType  # noqa: F401
from .collectives import (bind, log_uniform_sizes, ring_allreduce, ring_allreduce_signalled,  # noqa: F401
                          small_message_allreduce)  # noqa: F401
