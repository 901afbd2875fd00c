"""Tensor graph wiring, segmentation, nanobatch interleaving, slot naming — host logic only.
Expected values are hand-derived from the reference's rules (file:line in each test)."""

import pytest
import torch

from kareus_amd import LayerConfig, LayerStack
from kareus_amd.operators import (BiasDropoutAddOp, BiasSwigluOp, PartitionableRMSNorm, QKVPostProcessOp,
                                  ResidualForkOp, RotaryEmbeddingOp, TEColumnParallelLinearOp,
                                  TEDotProductAttentionOp, TERowParallelLinearOp)
from kareus_amd.partitions import (Channel, CommunicationOp, CommunicationOpSpec, CommunicationType,
                                   ComputeOp, ComputeOpSpec, PartitionableOperator, PartitionBuilder,
                                   TensorGraph, TensorGraphBuilder)
from kareus_amd.partitions.partition_base import _build_overlap_slots, _resolve_slot
from kareus_amd.scheduler import CommConfig


class _Op(PartitionableOperator):
    def __init__(self, ins=("main",), outs=("main",)):
        self._i, self._o = ins, outs

    def get_input_channels(self):
        return [Channel(i, n) for i, n in enumerate(self._i)]

    def get_output_channels(self):
        return [Channel(i, n) for i, n in enumerate(self._o)]

    def parameters(self):
        return []


def test_builder_ids_and_channel_persistence():
    # tensor_graph.py:233-283: ids t_0.., unknown inputs become ext_<name>, channels persist
    b = TensorGraphBuilder()
    b.add_initial_channels({"main": "ext_main"})
    split = b.add_op(ComputeOpSpec(_Op(outs=("main", "key", "value"))))
    rot = b.add_op(ComputeOpSpec(_Op(ins=("main", "key", "rotary_pos_emb"), outs=("main", "key"))))
    attn = b.add_op(ComputeOpSpec(_Op(ins=("main", "key", "value"))))
    assert split.get_input_tensor_ids() == ["ext_main"]
    assert split.get_output_tensor_ids() == ["t_0", "t_1", "t_2"]
    assert rot.get_input_tensor_ids() == ["t_0", "t_1", "ext_rotary_pos_emb"]
    assert rot.get_output_tensor_ids() == ["t_3", "t_4"]
    # "value" skipped over the rotary op untouched
    assert attn.get_input_tensor_ids() == ["t_3", "t_4", "t_2"]
    assert [split.op_id, rot.op_id, attn.op_id] == [0, 1, 2]
    g = b.build()
    assert g.get_output_channel("main") == "t_5" and g.get_output_channel("nope") is None


def test_backward_spec_reverses_and_prefixes_channels():
    # tensor_graph.py:178-188
    op = _Op(ins=("main", "key", "rotary_pos_emb"), outs=("main", "key"))
    spec = ComputeOpSpec(op, is_backward=True, op_id=7)
    assert [(c.port_idx, c.name) for c in spec.get_input_channels()] == [(0, "grad_main"), (1, "grad_key")]
    assert [c.name for c in spec.get_output_channels()] == ["grad_main", "grad_key", "grad_rotary_pos_emb"]
    b = TensorGraphBuilder()
    b.add_initial_channels({"grad_main": "ext_grad_main"})
    node = b.add_op(spec)
    assert node.op_id == 7 and node.get_input_tensor_ids() == ["ext_grad_main", "ext_grad_key"]


def test_comm_spec_reads_and_rewrites_same_channel():
    b = TensorGraphBuilder()
    b.add_initial_channels({"main": "ext_main"})
    b.add_op(ComputeOpSpec(_Op()))
    c = b.add_op(CommunicationOpSpec(CommunicationType.ALL_REDUCE, [Channel(0, "main")]))
    nxt = b.add_op(ComputeOpSpec(_Op()))
    assert isinstance(c, CommunicationOp) and c.get_input_tensor_ids() == ["t_0"]
    assert c.get_output_tensor_ids() == ["t_1"] and nxt.get_input_tensor_ids() == ["t_1"]
    with pytest.raises(RuntimeError):
        c.event_wait()  # no physical operator bound yet


def _ops(letters):
    out = []
    for ch in letters:
        if ch == "|":
            out.append(CommunicationOp(CommunicationType.ALL_REDUCE))
        else:
            out.append(ComputeOp(operator=ResidualForkOp(backend="eager"), op_id=len(out)))
    return out


def test_split_by_communications_docstring_example():
    # partition_builder.py:158-161: [A, AR, B, C, AR, D] -> ([A],AR), ([B,C],AR), ([D],None)
    ops = _ops("A|BC|D")
    segs = PartitionBuilder._split_by_communications(ops)
    assert [len(s[0]) for s in segs] == [1, 2, 1]
    assert segs[0][1] is ops[1] and segs[1][1] is ops[4] and segs[2][1] is None
    # a collective right after another replaces it on the closed segment (:174-178)
    ops = _ops("A||B")
    segs = PartitionBuilder._split_by_communications(ops)
    assert segs[0][1] is ops[2] and len(segs) == 2


def test_two_nanobatch_comm_assignment_rule():
    # partition_builder.py:89-95, 117-146
    ops = _ops("A|B|C")
    g = TensorGraph(ops=ops)
    parts = PartitionBuilder(g, g, 2).build_forward_partitions(["a", "a", "b", "b", "t", ""])
    assert [p.nano_batch_idx for p in parts] == [0, 1, 0, 1, 0, 1]
    assert [p.partition_id for p in parts] == list(range(6))
    assert parts[0].comm_op is None  # very first partition has nothing to hand over
    comm0, comm1 = ops[1], ops[3]
    same = lambda c, ref: c is not ref and c.input_ports is ref.input_ports and c.comm_type == ref.comm_type
    assert same(parts[1].comm_op, comm0)  # NB1 carries this segment's comm (NB0's tensor)
    assert same(parts[2].comm_op, comm0)  # NB0 carries the previous segment's comm (NB1's tensor)
    assert same(parts[3].comm_op, comm1) and same(parts[4].comm_op, comm1)
    assert parts[5].comm_op is None  # last segment has no comm after it
    assert parts[1].comm_op is not parts[2].comm_op  # independent operator slots
    with pytest.raises(RuntimeError, match="Partition key count mismatch"):
        PartitionBuilder(g, g, 2).build_forward_partitions(["a"] * 5)


def test_general_nanobatch_counts():
    ops = _ops("A|B|C")
    g = TensorGraph(ops=ops)
    p4 = PartitionBuilder(g, g, 4).build_backward_partitions(["k"] * 12)
    assert [p.nano_batch_idx for p in p4] == [0, 1, 2, 3] * 3
    assert [p.comm_op is None for p in p4] == [True] + [False] * 7 + [False] + [True] * 3
    # nanobatch 0 of segment 1 hands over the LAST nanobatch's segment-0 tensor
    assert p4[4].comm_op.input_ports is ops[1].input_ports and p4[5].comm_op.input_ports is ops[3].input_ports
    p1 = PartitionBuilder(g, g, 1).build_forward_partitions(["x", "y", "z"])
    assert [p.comm_op is None for p in p1] == [False, False, True]
    assert all(p.force_no_overlap for p in p1) and p1[0].comm_op.input_ports is ops[1].input_ports
    with pytest.raises(ValueError):
        PartitionBuilder(g, g, 0)


def _layer_ops():
    kw = dict(backend="eager", dtype=torch.float32)
    return dict(
        fork=ResidualForkOp(backend="eager"), ln=PartitionableRMSNorm(8, **kw),
        qkv=TEColumnParallelLinearOp(8, 16, **kw), post=QKVPostProcessOp(1, 2, 4), rope=RotaryEmbeddingOp(backend="eager"),
        attn=TEDotProductAttentionOp(backend="eager"), proj=TERowParallelLinearOp(8, 8, **kw),
        bda=BiasDropoutAddOp(backend="eager"), act=BiasSwigluOp(backend="eager"),
    )


def test_slot_names_match_reference_table():
    # partition_base.py:22-34 grouping, :58-63 merging; names used by the shipped schedules
    o = _layer_ops()
    mk = lambda names: [ComputeOp(operator=o[n], op_id=i) for i, n in enumerate(names)]
    fwd_attn_l2 = mk(["bda", "fork", "ln", "qkv", "post", "rope", "attn", "proj"])
    assert _build_overlap_slots(fwd_attn_l2) == {"norm_0": 0, "linear_0": 3, "rope_0": 4, "attn_0": 6, "linear_1": 7}
    fwd_attn_l1 = mk(["fork", "ln", "qkv", "post", "rope", "attn", "proj"])
    assert _build_overlap_slots(fwd_attn_l1) == {"norm_0": 0, "linear_0": 2, "rope_0": 3, "attn_0": 5, "linear_1": 6}
    fwd_mlp = mk(["bda", "fork", "ln", "qkv", "act", "proj"])
    assert _build_overlap_slots(fwd_mlp) == {"norm_0": 0, "linear_0": 3, "activation_0": 4, "linear_1": 5}
    bwd_attn = mk(["ln", "fork", "bda", "proj", "attn", "rope", "post", "qkv"])
    assert _build_overlap_slots(bwd_attn) == {"norm_0": 0, "linear_0": 3, "attn_0": 4, "rope_0": 5, "linear_1": 7}
    bwd_mlp = mk(["bda", "proj", "act", "qkv"])
    assert _build_overlap_slots(bwd_mlp) == {"norm_0": 0, "linear_0": 1, "activation_0": 2, "linear_1": 3}
    assert _resolve_slot({"norm_0": 0}, "none") == -1
    with pytest.raises(KeyError, match="Unknown overlap slot"):
        _resolve_slot({"norm_0": 0}, "attn_3")

    class Strange(torch.nn.Module):
        pass

    with pytest.raises(ValueError, match="Unknown operator class"):
        _build_overlap_slots([ComputeOp(operator=Strange(), op_id=0)])


def _stack(n_layers=2, nnb=2):
    cfg = LayerConfig(hidden_size=32, num_attention_heads=4, num_query_groups=2, kv_channels=8,
                      ffn_hidden_size=24, num_layers=n_layers, num_nanobatches=nnb,
                      params_dtype=torch.float32, backend="eager")
    return LayerStack(cfg, seed=3)


def test_stack_segments_keys_and_schedule_resolution():
    m = _stack(2, 2)
    fp, bp = m.forward_partitions, m.backward_partitions
    # 2*(2L+1) partitions per direction (transformer_block.py:205-212)
    assert len(fp) == len(bp) == 10
    assert [p.partition_key for p in fp] == ["fwd_attn"] * 2 + ["fwd_mlp"] * 2 + ["fwd_attn"] * 2 + ["fwd_mlp"] * 2 + ["fwd_trail", ""]
    assert [p.partition_key for p in bp] == ["bwd_mlp"] * 2 + ["bwd_attn"] * 2 + ["bwd_mlp"] * 2 + ["bwd_attn"] * 2 + ["bwd_trail", ""]
    names = lambda p: [type(o.operator).__name__ for o in p.comp_ops]
    assert names(fp[0]) == ["ResidualForkOp", "PartitionableRMSNorm", "TEColumnParallelLinearOp", "QKVPostProcessOp",
                            "RotaryEmbeddingOp", "TEDotProductAttentionOp", "TERowParallelLinearOp"]
    assert names(fp[2]) == ["BiasDropoutAddOp", "ResidualForkOp", "PartitionableRMSNorm", "TEColumnParallelLinearOp",
                            "BiasSwigluOp", "TERowParallelLinearOp"]
    assert names(fp[4])[0] == "BiasDropoutAddOp" and len(fp[4].comp_ops) == 8  # mlp_bda of layer 1 + attention of layer 2
    assert names(fp[8]) == ["BiasDropoutAddOp"]
    assert names(bp[0]) == ["BiasDropoutAddOp", "TERowParallelLinearOp", "BiasSwigluOp", "TEColumnParallelLinearOp"]
    assert names(bp[2]) == ["PartitionableRMSNorm", "ResidualForkOp", "BiasDropoutAddOp", "TERowParallelLinearOp",
                            "TEDotProductAttentionOp", "RotaryEmbeddingOp", "QKVPostProcessOp", "TEColumnParallelLinearOp"]
    assert names(bp[8]) == ["PartitionableRMSNorm", "ResidualForkOp"]
    # backward nodes reuse the forward op ids; parameter order == op id order
    fwd_ids = {id(o.operator): o.op_id for o in m.forward_tensor_graph.get_compute_ops()}
    assert all(fwd_ids[id(o.operator)] == o.op_id for o in m.backward_tensor_graph.get_compute_ops())
    assert len(m._get_all_params()) == 12
    # CommConfig(("rope_0","none"),(21,1024)) on a layer>=2 attention partition -> (4,-1,21,1024)
    class Item:
        fwd_attn = CommConfig(("rope_0", "none"), (21, 1024))
    fp[5].load_schedule(Item())
    assert fp[5]._get_comm_config() == ((4, -1), (21, 1024))
    fp[1].load_schedule(Item())
    assert fp[1]._get_comm_config() == ((3, -1), (21, 1024))  # first layer has no leading bda
    assert fp[3]._get_comm_config() == ((0, -1), (None, None))  # nothing loaded: default window
    # every hand-over slot of a non-first partition is bound to a schedule-point operator
    assert all(p.comm_op is None or p.comm_op.operator is not None for p in fp + bp)
    assert sum(p.comm_op is None for p in fp) == 2 and sum(p.comm_op is None for p in bp) == 2


def test_comm_end_must_be_none_sentinel():
    m = _stack(1, 2)
    class Item:
        fwd_attn = CommConfig((0, 3), (16, 1024))
        fwd_mlp = fwd_trail = None
    class Sch:
        current_schedule = Item()
    m.config.kareus_scheduler = Sch()
    with pytest.raises(ValueError, match="comm_end must be -1"):
        m(torch.randn(4, 2, 32))
