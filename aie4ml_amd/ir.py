"""Operator IR the GPU executor consumes.

Same shape as the reference's logical IR (src/aie4ml/ir/graph.py:16-348: TensorVar / OpNode /
TraitInstance / LogicalIR / ExecutionEntry) and backend context (src/aie4ml/ir/context.py:49-180), so
graphs lowered by the reference's ONNX / hls4ml frontends can be handed to this backend unchanged: the
passes and operator variants here only use attribute access on these objects.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Iterable, List, Optional, Sequence, Tuple

import numpy as np


@dataclass
class TensorVar:
    """A value in the graph. Parameters carry `data` (float64) and have no producer."""

    name: str
    shape: Tuple[int, ...]
    precision: Any = None
    data: Optional[np.ndarray] = None
    producer: Optional['OpNode'] = None
    consumers: List['OpNode'] = field(default_factory=list)

    @property
    def is_parameter(self) -> bool:
        return self.data is not None


@dataclass
class TraitInstance:
    name: str
    data: Dict[str, Any] = field(default_factory=dict)


@dataclass
class OpNode:
    name: str
    op_type: str
    dialect: str = 'CDNA'
    inputs: List[TensorVar] = field(default_factory=list)
    outputs: List[TensorVar] = field(default_factory=list)
    artifacts: Dict[str, Any] = field(default_factory=dict)
    traits: Dict[str, TraitInstance] = field(default_factory=dict)
    metadata: Dict[str, Any] = field(default_factory=dict)
    directives: Dict[str, Any] = field(default_factory=dict)
    roles: Dict[str, str] = field(default_factory=dict)
    is_placeholder: bool = False

    def add_trait(self, trait: TraitInstance) -> None:
        self.traits[trait.name] = trait

    def trait_data(self, name: str) -> Dict[str, Any]:
        t = self.traits.get(name)
        return t.data if t is not None else {}


def set_input_roles(node: OpNode, tensors: Sequence[TensorVar], role_names: Sequence[str]) -> None:
    if len(tensors) != len(role_names):
        raise ValueError(f'{node.name}: set_input_roles got {len(tensors)} tensors but {len(role_names)} role names.')
    node.roles = {t.name: str(r) for t, r in zip(tensors, role_names)}


def input_role(node: OpNode, tensor_name: str) -> Optional[str]:
    return node.roles.get(tensor_name)


def input_tensor_for_role(node: OpNode, role: str) -> TensorVar:
    for t in node.inputs:
        if node.roles.get(t.name) == role:
            return t
    raise ValueError(f'{node.name}: missing {role} tensor.')


def optional_tensor_for_role(node: OpNode, role: str) -> Optional[TensorVar]:
    for t in node.inputs:
        if node.roles.get(t.name) == role:
            return t
    return None


@dataclass
class LogicalIR:
    tensors: Dict[str, TensorVar] = field(default_factory=dict)
    nodes: List[OpNode] = field(default_factory=list)
    input_tensor_names: List[str] = field(default_factory=list)
    output_tensor_names: List[str] = field(default_factory=list)

    # ---- construction
    def add_tensor(self, tensor: TensorVar) -> None:
        if tensor.name in self.tensors:
            raise ValueError(f"Tensor '{tensor.name}' already exists.")
        self.tensors[tensor.name] = tensor

    def add_node(self, node: OpNode) -> None:
        self.nodes.append(node)

    def mark_graph_input(self, name: str) -> None:
        if name not in self.tensors:
            raise ValueError(f"Graph input tensor '{name}' does not exist.")
        if name not in self.input_tensor_names:
            self.input_tensor_names.append(name)

    def mark_graph_output(self, name: str) -> None:
        if name not in self.tensors:
            raise ValueError(f"Graph output tensor '{name}' does not exist.")
        if name not in self.output_tensor_names:
            self.output_tensor_names.append(name)

    def graph_inputs(self) -> List[TensorVar]:
        if not self.input_tensor_names:
            raise ValueError('LogicalIR.graph_inputs requires explicit input_tensor_names.')
        return [self.tensors[n] for n in self.input_tensor_names]

    def graph_outputs(self) -> List[TensorVar]:
        if not self.output_tensor_names:
            raise ValueError('LogicalIR.graph_outputs requires explicit output_tensor_names.')
        return [self.tensors[n] for n in self.output_tensor_names]

    # ---- surgery used by the fold / fuse passes
    def remove_node(self, node: OpNode, mode: str = 'bypass') -> None:
        """Cut a node out. 'bypass': consumers read the node's input instead of its output.
        'contract': the node's producer writes the node's output directly (single-consumer input only)."""
        if len(node.inputs) == 1 and len(node.outputs) == 1:
            src, dst = node.inputs[0], node.outputs[0]
            if mode == 'bypass':
                for consumer in list(dst.consumers):
                    consumer.inputs = [src if t is dst else t for t in consumer.inputs]
                    if consumer not in src.consumers:
                        src.consumers.append(consumer)
                    if dst.name in consumer.roles:
                        consumer.roles[src.name] = consumer.roles.pop(dst.name)
                if node in src.consumers:
                    src.consumers.remove(node)
                dst.producer = None
                dst.consumers.clear()
                self.tensors.pop(dst.name, None)
                if dst.name in self.output_tensor_names:  # a graph output that was only renamed
                    self.output_tensor_names[self.output_tensor_names.index(dst.name)] = src.name
            elif mode == 'contract':
                if len(src.consumers) != 1:
                    raise ValueError(f'Cannot contract node {node.name}: input tensor {src.name} has '
                                     f'{len(src.consumers)} consumers.')
                producer = src.producer
                if producer is not None:
                    producer.outputs = [dst if t is src else t for t in producer.outputs]
                dst.producer = producer
                src.consumers.remove(node)
                src.producer = None
                self.tensors.pop(src.name, None)
            else:
                raise ValueError(f'Unknown mode: {mode}')
        else:
            for t in node.inputs:
                if node in t.consumers:
                    t.consumers.remove(node)
            for t in node.outputs:
                if t.producer is node and t.consumers:
                    raise ValueError(f'Cannot detach node {node.name}: output tensor {t.name} still has consumers.')
                if t.producer is node:
                    t.producer = None
                    self.tensors.pop(t.name, None)
        if node in self.nodes:
            self.nodes.remove(node)
        node.inputs = []
        node.outputs = []

    # ---- invariants
    def verify(self) -> None:
        seen = set()
        for node in self.nodes:
            if node.name in seen:
                raise RuntimeError(f'LogicalIR has duplicate node name {node.name!r}.')
            for t in node.inputs:
                if t.is_parameter:
                    continue
                if t.producer is not None and t.producer.name not in seen:
                    raise RuntimeError(f'LogicalIR is not in topological order: {node.name!r} consumes {t.name!r} '
                                       f'whose producer {t.producer.name!r} has not yet been visited.')
                if t.producer is None and t.name not in self.input_tensor_names:
                    raise RuntimeError(f'{node.name}: activation input {t.name!r} has no producer and is not a '
                                       'declared graph input.')
            seen.add(node.name)

    def __iter__(self):
        return iter(self.nodes)

    def __len__(self):
        return len(self.nodes)


@dataclass
class ExecutionEntry:
    """A logical node bound to the operator variant that will run it, with its resolved constants."""

    node: OpNode
    variant: Any
    config: Any
    artifacts: Dict[str, Any] = field(default_factory=dict)

    @property
    def name(self) -> str:
        return self.node.name

    @property
    def op_type(self) -> str:
        return self.node.op_type


@dataclass
class ExecutionIR:
    instances: Dict[str, ExecutionEntry] = field(default_factory=dict)

    def register(self, node: OpNode, variant: Any, config: Any) -> ExecutionEntry:
        inst = ExecutionEntry(node=node, variant=variant, config=config)
        self.instances[node.name] = inst
        return inst

    def get(self, name: str) -> Optional[ExecutionEntry]:
        return self.instances.get(name)

    def prune(self, keep: Iterable[str]) -> bool:
        keep = set(keep)
        stale = [n for n in self.instances if n not in keep]
        for n in stale:
            del self.instances[n]
        return bool(stale)

    def __iter__(self):
        return iter(self.instances.values())


@dataclass
class PipelineIR:
    logical: LogicalIR = field(default_factory=LogicalIR)
    execution: ExecutionIR = field(default_factory=ExecutionIR)


@dataclass
class DeviceSpec:
    """The one device this backend targets; `generation` is what operator variants match on."""

    platform: str = 'mi355x'
    generation: str = 'CDNA4'
    arch: str = 'gfx950'
    compute_units: int = 256
    lds_bytes: int = 160 * 1024
    hbm_bytes: int = 288 * (1 << 30)


@dataclass
class BackendContext:
    """Container passed between passes (device, graph, run configuration)."""

    device: DeviceSpec = field(default_factory=DeviceSpec)
    config: Dict[str, Any] = field(default_factory=dict)
    ir: PipelineIR = field(default_factory=PipelineIR)


CONTEXT_ATTR = '_aie_backend_context'


def get_backend_context(model_or_ctx):
    """Accepts a context, or any model object carrying one (as the reference's passes do)."""
    if hasattr(model_or_ctx, 'ir') and hasattr(model_or_ctx, 'device'):
        return model_or_ctx
    ctx = getattr(model_or_ctx, CONTEXT_ATTR, None)
    if ctx is None:
        raise RuntimeError('AIE backend context missing. Run lowering before invoking downstream passes.')
    return ctx
