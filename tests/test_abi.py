"""The C-ABI library loads without a GPU and exports every symbol the header declares;
host-side logic (topology on the host, argument checks) behaves like the reference's."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import oracle
import sparseattention_amd as sa
from sparseattention_amd import _lib
from sparseattention_amd.ops import functional as fn
from sparseattention_amd.ops import topology as topo

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "hsa_gfx950.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hsa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.lib()
    names = declared_symbols()
    assert len(names) >= 9
    for n in names:
        assert hasattr(lib, n), "missing export " + n
    assert lib.hsa_abi_version() == 1


def test_public_names_match_reference_surface():
    for n in ["HierarchicalAttention", "build_tree_topology", "generate_span_input_Y",
              "build_parent_nodes", "hierarchical_attention", "__version__"]:
        assert hasattr(sa, n)


@pytest.mark.parametrize("N", [1, 2, 16, 512, 4096])
@pytest.mark.parametrize("causal", [True, False])
def test_host_topology_bit_exact(N, causal):
    t = sa.build_tree_topology(N, causal, device="cpu")
    o = oracle.topology_tables(N, causal)
    assert t["forward_idx"].dtype == torch.int32 and t["forward_mask"].dtype == torch.bool
    assert t["backward_gather"].dtype == torch.int32
    np.testing.assert_array_equal(t["forward_idx"].numpy(), o["forward_idx"])
    np.testing.assert_array_equal(t["forward_mask"].numpy(), o["forward_mask"])
    np.testing.assert_array_equal(t["backward_gather"].numpy(), o["backward_gather"])


def test_topology_rejects_non_power_of_two():
    with pytest.raises(AssertionError):
        sa.build_tree_topology(12, True, device="cpu")
    assert _lib.lib().hsa_topology_host(12, 1, None, None, None) == -22
    assert b"power of 2" in _lib.lib().hsa_last_error()


def test_topology_int64_dtype():
    t = sa.build_tree_topology(8, True, device="cpu", dtype=torch.int64)
    assert t["forward_idx"].dtype == torch.int64 and t["backward_gather"].dtype == torch.int64


def test_canonical_table_registry():
    t = sa.build_tree_topology(16, True, device="cpu")
    assert topo.known_table(t["forward_idx"], "idx") == (16, True)
    assert topo.known_table(t["forward_mask"], "mask") == (16, True)
    assert fn._is_canonical(t["forward_idx"], t["forward_mask"], 16) is True
    assert fn._is_canonical(t["forward_idx"], None, 16) is False
    clone = t["forward_idx"].clone()
    assert fn._is_canonical(clone, None, 16) is None          # unknown origin
    t["forward_idx"][0, 0] = 5                                  # in-place edit invalidates
    assert fn._is_canonical(t["forward_idx"], None, 16) is None


def test_attention_argument_checks_on_host():
    lib = _lib.lib()
    one = ctypes.c_void_p(16)
    # null pointers
    assert lib.hsa_attn_fwd(None, one, one, None, None, one, None, 1, 16, 31, 1, 64, 4, 1, 1, 2, 0, None) == -22
    # canonical table needs L == log2 N
    assert lib.hsa_attn_fwd(one, one, one, None, None, one, None, 1, 16, 31, 1, 64, 3, 1, 1, 2, 0, None) == -22
    # ... and M >= 2N-1
    assert lib.hsa_attn_fwd(one, one, one, None, None, one, None, 1, 16, 30, 1, 64, 4, 1, 1, 2, 0, None) == -22
    # unknown dtype
    assert lib.hsa_attn_fwd(one, one, one, None, None, one, None, 1, 16, 31, 1, 64, 4, 1, 1, 7, 0, None) == -22
    assert lib.hsa_build_parents_fwd(None, one, one, one, one, one, None, 1, 1, 1, 8, 0, 0, 0, 0, 0, 0, 0, None) == -22
    assert lib.hsa_build_tree_fwd(one, one, one, one, one, one, None, 1, 12, 1, 8, 0, 0, 0, 0, 0, 0, 0, 0, None) == -22
    assert lib.hsa_span_input_y(one, one, 1, 1, 4, 0, None) == -22


def test_ops_refuse_cpu_tensors_instead_of_falling_back():
    q = torch.randn(1, 4, 1, 8)
    k = torch.randn(1, 7, 1, 8)
    t = sa.build_tree_topology(4, True, device="cpu")
    with pytest.raises(_lib.HsaError):
        sa.hierarchical_attention(q, k, k, t["forward_idx"], t["backward_gather"], t["forward_mask"], 1)
    with pytest.raises(_lib.HsaError):
        sa.build_parent_nodes(q[:, :2], q[:, :2], q[:, :2], q, q)
    with pytest.raises(_lib.HsaError):
        sa.generate_span_input_Y(torch.randn(1, 4, 8))


def test_module_state_dict_names():
    m = sa.HierarchicalAttention(32, 4, dropout=0.0, window_size=2)
    keys = set(m.state_dict().keys())
    assert keys == {"Wq_y.weight", "Wk_y.weight", "Wv_y.weight", "out_proj_y.weight", "out_proj_y.bias",
                    "Wq_x.weight", "Wk_x.weight", "Wv_x.weight", "out_proj_x.weight", "out_proj_x.bias"}
    assert m._build_level_info(16) == ([8, 4, 2, 1], [0, 8, 12, 14])


def test_transformer_lm_state_dict_layout():
    m = sa.TransformerLM(50, 32, 4, 64, 1, dropout=0.0, max_len=64)
    keys = set(m.state_dict().keys())
    for k in ["embedding.weight", "pos_encoding.pe", "fc_out.weight", "fc_out.bias",
              "layers.0.self_attn.Wq_y.weight", "layers.0.self_attn.out_proj_x.bias",
              "layers.0.feed_forward.fc1.weight", "layers.0.norm_y.weight", "layers.0.alpha_proj.weight",
              "layers.0.beta_proj.bias"]:
        assert k in keys
    assert m.fc_out.weight is m.embedding.weight
    # a reference-style checkpoint with a DataParallel prefix loads
    ck = {"model_state_dict": {"module." + k: v for k, v in m.state_dict().items()}}
    m.load_reference_checkpoint(ck)
