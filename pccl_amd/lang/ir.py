"""Collective IR: the vocabulary of the reference's ``pccl/lang/chunk.py`` plus what the
executor needs to run it.

Kept from the reference: ``PrimitiveOpType`` (chunk.py:6-10), ``DeviceType`` (:12-15), ``Chunk``
(:17-30), ``Device`` (:32-37), ``Link`` (:39-44), ``PrimitiveOp`` (:46-55) and the
``CollectiveIR`` container with ``create_operation`` / ``validate_dag`` /
``get_operation_sequence`` (:57-135).  ``Chunk.data_size`` and ``Chunk.offset`` count ELEMENTS
of the collective's dtype inside the per-device buffer named by ``metadata``.

Added, because the reference stops at the container: REDUCE ops may name extra sources and
destinations in ``metadata`` (``srcs`` / ``dsts``: lists of ``(buffer, device, offset)``), which
is the multi-input / multi-output form the executors run, and :meth:`CollectiveIR.lower` turns
the IR into the operand-level op list of the C ABI (``pccl_op_desc``).
"""
from dataclasses import dataclass, field
from enum import Enum, auto
from typing import Any, Dict, List, Optional, Set

from .graph import DirectedGraph


class PrimitiveOpType(Enum):
    COPY = auto()
    REDUCE = auto()
    NOTIFY = auto()
    GET_NOTIFIED = auto()


class DeviceType(Enum):
    CUDA = auto()
    CPU = auto()
    ROCM = auto()


@dataclass
class Chunk:
    reduced_ranks: Set[int]
    cur_device_id: int
    data_size: int
    offset: int

    def copy(self):
        return Chunk(set(self.reduced_ranks), self.cur_device_id, self.data_size, self.offset)


@dataclass
class Device:
    device_id: int
    device_type: DeviceType
    memory_bandwidth: float
    compute_capability: float


@dataclass
class Link:
    src_device: int
    dst_device: int
    bandwidth: float
    latency: float


@dataclass
class PrimitiveOp:
    op_type: PrimitiveOpType
    op_id: int
    src_chunk: Optional[Chunk]
    tgt_chunk: Optional[Chunk]
    src_device: Optional[int]
    tgt_device: Optional[int]
    dependencies: List[int]
    metadata: Dict[str, Any] = field(default_factory=dict)


class CollectiveIR:
    def __init__(self, name: str, dtype: str = "bf16", compute: str = "sum"):
        self.name = name
        self.dtype = dtype
        self.compute = compute
        self.precondition: List[Chunk] = []
        self.postcondition: List[Chunk] = []
        self.devices: Dict[int, Device] = {}
        self.links: List[Link] = []
        self.ops: Dict[int, PrimitiveOp] = {}
        self.op_dag = DirectedGraph()
        self.device_topology = DirectedGraph()
        self._next_op_id = 0

    # -- topology -------------------------------------------------------------------------
    def add_device(self, device: Device):
        # the topology graph numbers nodes densely in insertion order (graph.py:23-27), so
        # device ids must be 0, 1, 2, ... in the order they are added
        expected = self.device_topology.num_nodes()
        if device.device_id != expected:
            raise ValueError("device ids must be dense and added in order (got %d, expected %d)"
                             % (device.device_id, expected))
        self.device_topology.add_node(device.device_id)
        self.devices[device.device_id] = device

    def add_link(self, link: Link):
        self.links.append(link)
        self.device_topology.add_edge(link.src_device, link.dst_device)
        self.device_topology.add_edge(link.dst_device, link.src_device)

    # -- ops ------------------------------------------------------------------------------
    def create_operation(self, op_type, src_chunk=None, tgt_chunk=None, src_device=None, tgt_device=None,
                         dependencies=None, metadata=None) -> int:
        op_id = self._next_op_id
        self._next_op_id += 1
        op = PrimitiveOp(op_type, op_id, src_chunk, tgt_chunk, src_device, tgt_device,
                         list(dependencies or []), dict(metadata or {}))
        self.ops[op_id] = op
        self.op_dag.add_node(op_id)
        for dep in op.dependencies:
            self.op_dag.add_edge(dep, op_id)
        return op_id

    def set_precondition(self, chunks):
        self.precondition = chunks

    def set_postcondition(self, chunks):
        self.postcondition = chunks

    def validate_topology(self) -> bool:
        return len(self.device_topology.get_connected_components()) == 1

    def validate_dag(self) -> bool:
        return self.op_dag.is_acyclic()

    def get_device_bandwidth_matrix(self):
        m = {}
        for l in self.links:
            m[(l.src_device, l.dst_device)] = l.bandwidth
            m[(l.dst_device, l.src_device)] = l.bandwidth
        return m

    def get_operation_sequence(self) -> List[PrimitiveOp]:
        try:
            return [self.ops[i] for i in self.op_dag.topological_sort()]
        except ValueError:
            return []

    # -- the engine's schedule file -------------------------------------------------------
    def serialize(self, elems_per_device=None):
        """Text of the schedule file ``Engine.regOp(name, filepath)`` loads (format documented
        in ``pccl_amd/csrc/host/schedule.h``)."""
        low = self.lower()
        if elems_per_device is None:
            elems_per_device = max([x[2] + o["count"] for o in low for x in o["ins"] + o["outs"] if x[0] != "ws"] or [0])
        by_part = any(o["primitive"] >= 2 and o.get("parts", 1) > 1 for o in low)   # only format version 2 can say that
        lines = ["pccl-schedule %d" % (2 if by_part else 1), "name %s" % (self.name.replace(" ", "_") or "unnamed"), "dtype %s" % self.dtype,
                 "compute %s" % self.compute, "devices %d" % max(len(self.devices), 1),
                 "elems_per_device %d" % elems_per_device, "ops %d" % len(low)]
        kinds = ("COPY", "REDUCE", "NOTIFY", "GET_NOTIFIED")
        for i, o in enumerate(low):
            parts = ["op %d %s %d deps %d" % (i, kinds[o["primitive"]], o["count"], len(o["deps"]))]
            parts += [str(d) for d in o["deps"]]
            if o["primitive"] >= 2:
                lines.append(" ".join(parts + ["slot %d" % o["slot"]] + (["parts %d" % o.get("parts", 1)] if by_part else [])))
                continue
            for key, ops in (("src", o["ins"]), ("dst", o["outs"])):
                parts.append("%s %d" % (key, len(ops)))
                parts += ["%s %d %d" % (b, dev, off) for (b, dev, off) in ops]
            lines.append(" ".join(parts))
        return "\n".join(lines) + "\n"

    def save(self, path, elems_per_device=None):
        with open(path, "w") as f:
            f.write(self.serialize(elems_per_device))

    # -- lowering to operand level --------------------------------------------------------
    def lower(self):
        """Returns a list of dicts (dtype, compute, primitive, ins, outs, count, deps) whose
        operands are symbolic ``(buffer, device, element_offset)`` triples, op ids preserved.

        NOTIFY / GET_NOTIFIED lower to signal ops (``primitive`` 2 / 3, ``slot``, ``value``, ``parts``: slots the
        signal takes, one per part of the data it announces; metadata "parts", default 1).
        A COPY reads ``src_chunk`` and writes ``tgt_chunk``.  A REDUCE folds its sources in
        order and writes every destination; without ``metadata["srcs"]`` it is the reference's
        two-operand form "reduce src into tgt": fold(src, tgt) -> tgt."""
        out = []
        for op_id in range(self._next_op_id):
            op = self.ops[op_id]
            md = op.metadata
            if op.op_type in (PrimitiveOpType.NOTIFY, PrimitiveOpType.GET_NOTIFIED):
                # signal ops name a workspace signal slot and a value (metadata "slot", "value")
                if "slot" not in md or "value" not in md:
                    raise ValueError("op %d: NOTIFY / GET_NOTIFIED need metadata 'slot' and 'value'" % op_id)
                prim = 2 if op.op_type is PrimitiveOpType.NOTIFY else 3
                out.append(dict(primitive=prim, slot=int(md["slot"]), value=int(md["value"]), ins=[], outs=[],
                                count=int(md["value"]), deps=list(op.dependencies), parts=int(md.get("parts", 1))))
                continue
            src = (md.get("src_buffer", "out"), op.src_device, op.src_chunk.offset)
            tgt = (md.get("tgt_buffer", "out"), op.tgt_device, op.tgt_chunk.offset)
            if op.op_type is PrimitiveOpType.COPY:
                ins, outs, prim = [src], [tgt] + list(md.get("dsts", [])), 0
            else:
                ins = list(md["srcs"]) if "srcs" in md else [src, tgt]
                outs, prim = [tgt] + list(md.get("dsts", [])), 1
            out.append(dict(dtype=self.dtype, compute=self.compute, primitive=prim, ins=ins, outs=outs,
                            count=op.tgt_chunk.data_size, deps=list(op.dependencies)))
        return out
