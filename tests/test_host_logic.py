"""Host-side logic that needs no GPU: workloads, the wire-format planner, the
mirrored module's construction and its refusal to run anywhere but on the GPU."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O


def test_workloads_are_seeded_and_shaped():
    from ccfuser_amd.workloads import make_workload, WORKLOAD_NAMES
    assert WORKLOAD_NAMES == ("c1_tiny", "c2_gshard", "c3_mixtral", "c4_ep_share", "c5_skewed")
    a, b = make_workload("c1_tiny"), make_workload("c1_tiny")
    for k in a.tensors:
        assert torch.equal(a.tensors[k], b.tensors[k])
    assert a.tensors["x"].shape == (512, 256) and a.tensors["x"].dtype == torch.float32
    assert a.tensors["w1"].shape == (4, 1024, 256) and a.tensors["w2"].shape == (4, 256, 1024)
    c2 = make_workload("c2_gshard", scale_rows=64)
    assert c2.capacity == int(np.ceil(1.25 * 64 * 2 / 8)) and c2.tensors["x"].dtype == torch.float16
    assert make_workload("c2_gshard", scale_rows=8192).capacity == 2560
    assert abs(c2.flops(100) - 4 * 100 * 1024 * 4096) < 1


def test_ep_share_segments_are_well_formed():
    from ccfuser_amd.workloads import make_workload
    wl = make_workload("c4_ep_share", scale_rows=2048)
    t = wl.tensors
    st, ln, ex, src = (t[n].tolist() for n in ("seg_start", "seg_len", "seg_expert", "seg_source"))
    assert len(st) <= 64 and sum(ln) == 2048
    at = 0
    for s, l in zip(st, ln):                   # contiguous cover of the inbound buffer
        assert s == at and l > 0
        at += l
    assert len(set(src)) == 8 and src == sorted(src)
    for s in range(8):                          # inside a source, grouped by local expert
        es = [e for e, q in zip(ex, src) if q == s]
        assert es == sorted(es) and len(set(es)) == len(es)


def test_skewed_workload_has_tiny_experts():
    from ccfuser_amd.workloads import make_workload
    wl = make_workload("c5_skewed", scale_rows=8192)
    t = wl.tensors
    idx = (t["x"].float() @ t["wg"].float().t() + t["bg"].float()).argmax(1)
    cnt = torch.bincount(idx, minlength=32)
    assert (cnt <= 16).sum() >= 3 and cnt.max() > 0.3 * 8192


def test_product_planner_matches_oracle_planner():
    from ccfuser_amd.mix_moe.transformer import plan_blocks
    g = np.random.default_rng(0)
    for _ in range(20):
        counts = (g.integers(0, 400, size=g.integers(1, 40)) * (g.random(1) < 0.9)).tolist()
        if sum(counts) == 0:
            continue
        a, b = plan_blocks(counts), O.divide_into_block(counts)
        assert a == b


def test_module_construction_and_state_dict_names():
    from ccfuser_amd.mix_moe import MixMOETransformerMLP, NaiveGate
    seen = []
    mlp = MixMOETransformerMLP("naive", {"num_local_expert": 4, "hidden_size": 128}, 64, 0, 1,
                               scan_expert_func=lambda n, p: seen.append(n), total_batch_size=256)
    assert sorted(mlp.state_dict()) == ["experts.h4toh.bias", "experts.h4toh.weight",
                                        "experts.htoh4.bias", "experts.htoh4.weight",
                                        "gate.gate.bias", "gate.gate.weight"]
    # E + 3 expert slots like the reference (transformer.py:449-453), [E, out, in] layout
    assert mlp.experts.htoh4.weight.shape == (7, 128, 64) and mlp.experts.h4toh.weight.shape == (7, 64, 128)
    assert sorted(seen) == ["h4toh.bias", "h4toh.weight", "htoh4.bias", "htoh4.weight"]
    assert all(p.dp_comm == "none" for p in mlp.experts.parameters())
    assert all(p.dp_comm == "gate" for p in mlp.gate.parameters())
    assert isinstance(mlp.gate, NaiveGate) and mlp.top_k == 2
    with pytest.raises(NotImplementedError):
        MixMOETransformerMLP("naive", {"num_local_expert": 4, "hidden_size": 128}, 64, 0, 2)
    with pytest.raises(TypeError):
        mlp(torch.randn(4, 64))                         # fp32: the GPU path is fp16 only
    with pytest.raises(ValueError, match="no CPU path"):
        mlp.half()(torch.randn(4, 64).half())           # CPU tensor: refuses, no fallback
    mlp.close()


def test_functions_refuse_multi_gpu():
    from ccfuser_amd.mix_moe import functions
    with pytest.raises(NotImplementedError):
        functions.count_by_gate(torch.zeros(4, dtype=torch.long), 2, 2, 0)
    with pytest.raises(RuntimeError):
        functions.ensure_comm(torch.zeros(1), object())


def test_integration_guide_constructor_example_is_valid():
    """The constructor call INTEGRATION.md shows for replacing the layer (the reference's
    positional order, transformer.py:435-461) must be accepted as written."""
    import os
    import re
    from ccfuser_amd.mix_moe import MixMOETransformerMLP
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    m = re.search(r"mlp = (MixMOETransformerMLP\(.*?\))\.cuda\(\)", text, flags=re.S)
    assert m, "the guide no longer shows the constructor call"
    mlp = eval(m.group(1), {"MixMOETransformerMLP": MixMOETransformerMLP})
    assert mlp.experts.htoh4.weight.shape[1:] == (14336, 4096) and mlp.top_k == 2
