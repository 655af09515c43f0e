"""Python collective IR (the reference's ``pccl/lang``) and schedule emitters."""
from .graph import DirectedGraph  # noqa: F401
from .ir import Chunk, CollectiveIR, Device, DeviceType, Link, PrimitiveOp, PrimitiveOpType  # noqa: F401
from .collectives import (ELEM_BYTES, all_to_all, bind, broadcast, direct_allreduce, log_uniform_sizes,  # noqa: F401
                          ring_all_gather, ring_allreduce, ring_allreduce_signalled, ring_rank_share,  # noqa: F401
                          ring_reduce_scatter, small_message_allreduce)  # noqa: F401
