"""Channel-routed dataflow graph for the partition engine.

Operators never name each other.  Each one declares the *channels* it reads and
writes ("main", "key", "residual", ...); the builder keeps a channel -> tensor-id
table that survives from op to op, so a value written early (``value`` by the QKV
split, ``residual`` by the fork) reaches a later consumer without the ops in
between knowing about it.  Tensor ids (``t_<n>``, ``ext_<channel>``) are the keys
of the per-nanobatch ``TensorStore`` at run time.

Behavioural contract follows kareus/megatron/core/partitions/tensor_graph.py
(reference): id numbering ``:233-241``, input wiring with ``ext_`` fallback and
output registration ``:255-283``, op_id assignment ``:286-287``, backward channel
derivation (``grad_`` prefix, inputs and outputs swapped) ``:178-188``,
communication specs reading and writing the same channels ``:203-207``, comm-op
delegation to a late-bound operator ``:111-121``.
"""

from __future__ import annotations

import enum
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence, Union


class CommunicationType(enum.Enum):
    """Kinds of collective a graph may place between partitions."""

    ALL_REDUCE = enum.auto()
    ALL_GATHER_KV = enum.auto()
    REDUCE_SCATTER_KV = enum.auto()


@dataclass
class Channel:
    """A named endpoint of an operator; ``port_idx`` is its positional slot."""

    port_idx: int
    name: str


@dataclass
class TensorPort:
    """One wired endpoint: positional slot plus the tensor id bound to it."""

    port_idx: int
    tensor_id: Optional[str] = None


def _ids(ports: Sequence[TensorPort]) -> List[Optional[str]]:
    return [port.tensor_id for port in ports]


@dataclass
class ComputeOp:
    """A compute node.  ``op_id`` keys the per-op context shared by fwd and bwd."""

    operator: Any
    input_ports: List[TensorPort] = field(default_factory=list)
    output_ports: List[TensorPort] = field(default_factory=list)
    op_id: int = -1

    def get_input_tensor_ids(self) -> List[Optional[str]]:
        return _ids(self.input_ports)

    def get_output_tensor_ids(self) -> List[Optional[str]]:
        return _ids(self.output_ports)


@dataclass
class CommunicationOp:
    """A collective node.  The physical operator is bound after graph build; the
    four protocol calls used by partitions are forwarded to it."""

    comm_type: CommunicationType
    input_ports: List[TensorPort] = field(default_factory=list)
    output_ports: List[TensorPort] = field(default_factory=list)
    operator: Optional[Any] = None

    def get_input_tensor_ids(self) -> List[Optional[str]]:
        return _ids(self.input_ports)

    def get_output_tensor_ids(self) -> List[Optional[str]]:
        return _ids(self.output_ports)

    def _bound(self):
        if self.operator is None:
            raise RuntimeError(
                f"CommunicationOp({self.comm_type.name}) has no physical operator bound"
            )
        return self.operator

    def event_record(self, stream) -> None:
        self._bound().event_record(stream)

    def event_wait(self) -> None:
        self._bound().event_wait()

    def fuser_forward(self, *args, **kwargs):
        return self._bound().fuser_forward(*args, **kwargs)

    def sync(self, stream) -> None:
        self._bound().sync(stream)


@dataclass
class ComputeOpSpec:
    """Request to add a compute node.

    With ``is_backward`` the channels are derived from the forward declaration:
    the node reads ``grad_<forward outputs>`` and writes ``grad_<forward inputs>``,
    ports renumbered from zero.  Explicit ``input_channels``/``output_channels``
    override what the operator declares.
    """

    operator: Any
    is_backward: bool = False
    op_id: Optional[int] = None
    input_channels: Optional[List[Channel]] = None
    output_channels: Optional[List[Channel]] = None

    def _fwd_in(self) -> List[Channel]:
        return self.input_channels or self.operator.get_input_channels()

    def _fwd_out(self) -> List[Channel]:
        return self.output_channels or self.operator.get_output_channels()

    @staticmethod
    def _as_grads(channels: Sequence[Channel]) -> List[Channel]:
        return [Channel(i, "grad_" + ch.name) for i, ch in enumerate(channels)]

    def get_input_channels(self) -> List[Channel]:
        return self._as_grads(self._fwd_out()) if self.is_backward else self._fwd_in()

    def get_output_channels(self) -> List[Channel]:
        return self._as_grads(self._fwd_in()) if self.is_backward else self._fwd_out()


@dataclass
class CommunicationOpSpec:
    """Request to add a collective node; it reads and rewrites ``channels``."""

    comm_type: CommunicationType
    channels: List[Channel] = field(default_factory=list)

    def get_input_channels(self) -> List[Channel]:
        return self.channels

    def get_output_channels(self) -> List[Channel]:
        return self.channels


class PartitionableOperator:
    """Mixin for operators the engine can place in a graph.

    Defaults describe a one-in/one-out op on ``main`` with a single compute node
    per direction.  Operators that own a collective (row-parallel linear forward,
    column-parallel linear backward) override ``get_forward_ops`` /
    ``get_backward_ops`` to append a ``CommunicationOpSpec``.
    """

    def get_forward_ops(self) -> List[Union[ComputeOpSpec, CommunicationOpSpec]]:
        return [ComputeOpSpec(operator=self)]

    def get_backward_ops(self) -> List[Union[ComputeOpSpec, CommunicationOpSpec]]:
        return [ComputeOpSpec(operator=self, is_backward=True)]

    def get_input_channels(self) -> List[Channel]:
        return [Channel(0, "main")]

    def get_output_channels(self) -> List[Channel]:
        return [Channel(0, "main")]


@dataclass
class TensorGraph:
    """Ordered nodes plus the final channel -> tensor-id table."""

    ops: List[Union[ComputeOp, CommunicationOp]] = field(default_factory=list)
    channel_registry: Dict[str, str] = field(default_factory=dict)

    def get_compute_ops(self) -> List[ComputeOp]:
        return [n for n in self.ops if isinstance(n, ComputeOp)]

    def get_comm_ops(self) -> List[CommunicationOp]:
        return [n for n in self.ops if isinstance(n, CommunicationOp)]

    def get_output_channel(self, channel_name: str) -> Optional[str]:
        return self.channel_registry.get(channel_name)


class TensorGraphBuilder:
    """Accumulates nodes while tracking which tensor id each channel holds."""

    def __init__(self) -> None:
        self._channel_registry: Dict[str, str] = {}
        self._ops: List[Union[ComputeOp, CommunicationOp]] = []
        self._tensor_counter = 0
        self._op_id_counter = 0

    def add_initial_channels(self, channels: Dict[str, str]) -> None:
        """Bind channels to externally provided tensors before any op is added."""
        self._channel_registry.update(channels)

    def _wire_inputs(self, channels: Sequence[Channel]) -> List[TensorPort]:
        ports = []
        for ch in channels:
            # A channel nobody has written yet is an external input of the graph.
            tid = self._channel_registry.setdefault(ch.name, "ext_" + ch.name)
            ports.append(TensorPort(ch.port_idx, tid))
        return ports

    def _wire_outputs(self, channels: Sequence[Channel]) -> List[TensorPort]:
        ports = []
        for ch in channels:
            tid = f"t_{self._tensor_counter}"
            self._tensor_counter += 1
            self._channel_registry[ch.name] = tid
            ports.append(TensorPort(ch.port_idx, tid))
        return ports

    def add_op(
        self, spec: Union[ComputeOpSpec, CommunicationOpSpec]
    ) -> Union[ComputeOp, CommunicationOp]:
        """Wire ``spec`` into the graph (inputs first, then fresh output ids)."""
        ins = self._wire_inputs(spec.get_input_channels())
        outs = self._wire_outputs(spec.get_output_channels())
        if isinstance(spec, ComputeOpSpec):
            if spec.op_id is None:
                op_id = self._op_id_counter
                self._op_id_counter += 1
            else:
                op_id = spec.op_id
            node: Union[ComputeOp, CommunicationOp] = ComputeOp(
                operator=spec.operator, input_ports=ins, output_ports=outs, op_id=op_id
            )
        else:
            node = CommunicationOp(comm_type=spec.comm_type, input_ports=ins, output_ports=outs)
        self._ops.append(node)
        return node

    def get_channel_registry(self) -> Dict[str, str]:
        return dict(self._channel_registry)

    def build(self) -> TensorGraph:
        return TensorGraph(ops=list(self._ops), channel_registry=dict(self._channel_registry))
