"""CPU-side checks: the C-ABI library loads and exports every symbol include/picomoe.h declares, host
logic (capacity, module structure, refusal of CPU tensors).  No kernels run here."""

import os
import re
import types

import ctypes

import pytest
import torch

from picotron_amd import _lib


def _declared_symbols():
    text = open(_lib.HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(picomoe_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 18
    for name in declared:
        assert hasattr(lib, name), name
    assert set(_lib.exported_symbols()) == set(declared)      # the ctypes table and the header agree
    assert lib.picomoe_abi_version() == _lib.ABI_VERSION
    assert b"unsupported" in lib.picomoe_error_string(1)
    assert lib.picomoe_error_string(0) == b"ok"


def test_argument_errors_are_reported_without_a_gpu():
    lib = _lib.load()
    null = None
    assert lib.picomoe_fp8_quant(null, 7, 4, 8, null, null, null) == 1           # bad dtype
    assert lib.picomoe_fp8_quant(null, 1, 4, 0, null, null, null) == 1           # bad width
    assert lib.picomoe_fp8_quant(null, 1, 0, 8, null, null, null) == 0           # empty input is fine
    assert lib.picomoe_route_fwd(null, 1, 4, 2000, 2, null, 1, null, null, null, null, null, null) == 1   # too many experts
    assert lib.picomoe_route_fwd(null, 1, 4, 8, 9, null, 1, null, null, null, null, null, null) == 1      # top_k > E
    assert lib.picomoe_permute_workspace_bytes(1000, 8) > 0
    assert lib.picomoe_permute_workspace_bytes(1000, 5000) == -1
    assert lib.picomoe_route_partials(8192, 8) >= 1
    # scratch of the split last round: 8 XCDs x 32 partial tiles of 256 x 256 fp32; empty inputs return before any launch
    assert lib.picomoe_ffn_workspace_bytes() == 8 * 32 * 256 * 256 * 4
    counts = ctypes.c_void_p(64)   # never dereferenced on the host: these calls return before any launch
    assert lib.picomoe_ffn_down(null, counts, 4, 0, 256, 128, null, null, 1, null, null, 0, null) == 0
    assert lib.picomoe_ffn_dgrad_x(null, counts, 4, 0, 256, 128, null, null, 1, null, null, 0, null) == 0
    assert lib.picomoe_ffn_down(null, counts, 4, 8, 256, 128, null, null, 1, null, null, 0, null) == 1    # null tensors
    assert lib.picomoe_ffn_down(null, null, 4, 0, 256, 128, null, null, 1, null, null, 0, null) == 1      # null counts
    # shapes whose tiles cannot be numbered in 32 bits are refused (PICOMOE_ERR_TOO_LARGE = 2) before anything is touched
    big_rows, big_width = 2**31 - 1, 2**24
    assert lib.picomoe_ffn_gate_up(null, counts, 4, big_rows, 256, big_width, null, null, 1, null, null, null, 0, null) == 2
    assert lib.picomoe_ffn_dgrad_x(null, counts, 4, big_rows, big_width, 256, null, null, 1, null, null, 0, null) == 2
    assert lib.picomoe_ffn_wgrad(counts, 2**26, counts, 2**26, counts, 1024, 8, 2**26, 2**26, 1, counts, null) == 2
    # diagnostics and queries
    assert lib.picomoe_diag_mfma_loop_flop(0, 10, 2) == 64 * 2 * 16 * 16 * 32 * 8 * 10 * 2
    assert lib.picomoe_diag_mfma_loop_flop(9, 10, 2) == -1
    assert lib.picomoe_diag_mfma_loop(null, 1024, 0, 10, 0, 0, 1, null, null) == 1                         # null operands
    assert lib.picomoe_dispatch_fp8(null, 1, 0, 64, null, 2, 0, null, null, null, null, null, null) == 0   # no tokens
    assert lib.picomoe_dispatch_fp8(null, 1, 4, 64, null, 17, 8, null, null, null, null, null, null) == 1  # top_k > 16
    assert lib.picomoe_dispatch_fp8(null, 1, 4, 64, null, 2, 8, null, counts, null, null, null, null) == 1 # codes without scales
    a16 = ctypes.c_void_p(64)
    assert lib.picomoe_gate_bwd(null, null, null, null, 1, 0, 8, 4096, null, null, null, 0, null) == 0            # no tokens, no d_w
    assert lib.picomoe_gate_bwd(a16, a16, null, null, 1, 4, 17, 4096, a16, null, null, 0, null) == 1             # more than 16 experts
    assert lib.picomoe_gate_bwd(a16, a16, null, a16, 1, 4, 9, 4096, a16, a16, a16, 1 << 30, null) == 1           # d_w with more than 8
    assert lib.picomoe_gate_bwd(a16, a16, null, null, 1, 4, 8, 4100, a16, null, null, 0, null) == 1              # row not in 16-byte chunks
    assert lib.picomoe_gate_bwd(a16, a16, ctypes.c_void_p(72), null, 0, 4, 8, 64, a16, null, null, 0, null) == 1 # misaligned addend
    assert lib.picomoe_gate_bwd(a16, a16, null, a16, 1, 4, 8, 4096, a16, a16, a16, 16, null) == 1                # workspace too small
    assert lib.picomoe_gate_bwd_workspace_bytes(1, 8192, 8, 4096) == 96 * 8 * 4096 * 4
    assert lib.picomoe_gate_bwd_workspace_bytes(0, 10, 4, 64) == 3 * 4 * 64 * 4          # three groups of four tokens
    assert lib.picomoe_gate_bwd_workspace_bytes(1, 8192, 9, 4096) == 0 and lib.picomoe_gate_bwd_workspace_bytes(2, 1, 1, 1) == -1
    assert lib.picomoe_ffn_kernel_family(1, 4096, 14336) == 1 and lib.picomoe_ffn_kernel_family(0, 256, 512) == 2
    assert lib.picomoe_ffn_kernel_family(1, 100, 36) == 0 and lib.picomoe_ffn_kernel_family(0, 16, 32) == 0
    assert b"fixed scratch" in lib.picomoe_error_string(2) and b"tile numbering" in lib.picomoe_error_string(2)
    with pytest.raises(_lib.PicomoeError):
        _lib.check(1, "demo")


def test_compute_capacity_matches_reference_table():
    from picotron_amd.expert_parallel.capacity_moe import compute_capacity

    assert [compute_capacity(512, 2, 8, f) for f in (0.5, 1.0, 1.25, 2.0)] == [64, 128, 160, 256]
    assert compute_capacity(16384, 6, 64, 1.25) == 1920
    assert compute_capacity(3, 1, 64, 0.1) == 1


def _cfg(**kw):
    base = dict(hidden_size=16, intermediate_size=32, num_experts=4, num_experts_per_tok=2)
    base.update(kw)
    return types.SimpleNamespace(**base)


def test_module_structure_and_defaults():
    from picotron_amd.expert_parallel.expert_parallel import MoELayer, collect_aux_loss

    moe = MoELayer(_cfg(num_shared_experts=2, moe_latent_dim=8, router_bias_update_rate=0.01))
    assert moe.expert_dim == 8 and moe.latent and moe.use_loss_free
    assert moe.local_experts[0].gate_proj.weight.shape == (32, 8)
    assert moe.shared_expert.gate_proj.weight.shape == (64, 16)
    assert moe.down_proj_latent.weight.shape == (8, 16) and moe.up_proj_latent.weight.shape == (16, 8)
    assert moe.expert_bias.shape == (4,) and "expert_bias" in moe.state_dict()
    plain = MoELayer(_cfg())
    assert plain.shared_expert is None and not plain.latent and plain.norm_topk_prob
    assert (plain.ep_capacity_factor, plain.ep_capacity_dropless, plain.ep_max_rounds) == (0.0, True, 8)
    assert plain.ep_fp8_dispatch is False and plain.router_aux_loss_coef == 0.0 and plain.aux_loss is None
    assert plain.ep_world_size == 1 and plain.num_local_experts == 4
    assert collect_aux_loss(plain) is None
    # default init: uniform in +-1/sqrt(fan_in), like the reference MLP
    w = plain.local_experts[0].down_proj.weight
    assert w.abs().max() <= (1.0 / 32) ** 0.5


def test_parameter_names_fit_the_reference_model_code():
    """The layer sits under ``DecoderLayer.mlp`` (model.py:306); the reference's parameter counting keys on the
    substrings ``mlp.local_experts.`` / ``mlp.gate.`` / ``mlp.shared_expert.`` (utils.py:82-86) and its checkpoint
    loader fills parameters missing from a dense checkpoint with zeros and then calls ``reset_parameters()``
    (checkpoint.py:132-141)."""
    from picotron_amd.expert_parallel.expert_parallel import MoELayer
    from picotron_amd.model import MLP

    class Block(torch.nn.Module):
        def __init__(self, cfg):
            super().__init__()
            self.mlp = MoELayer(cfg) if getattr(cfg, "num_experts", 1) > 1 else MLP(cfg)

    block = Block(_cfg(num_shared_experts=1))
    names = [n for n, _ in block.named_parameters()]
    experts = [n for n in names if "mlp.local_experts." in n]
    router = [n for n in names if "mlp.gate." in n]
    shared = [n for n in names if "mlp.shared_expert." in n]
    assert len(experts) == 4 * 3 and router == ["mlp.gate.weight"] and len(shared) == 3
    assert sorted(experts + router + shared) == sorted(names)
    assert "mlp.local_experts.2.up_proj.weight" in names and "mlp.expert_bias" in block.state_dict()
    # the zero-fill path: zeros in, proper init out
    sd = {n: torch.zeros(p.shape) for n, p in block.named_parameters()}
    sd["mlp.expert_bias"] = torch.zeros(4)
    block.load_state_dict(sd)
    assert all(float(p.detach().abs().sum()) == 0.0 for p in block.parameters())
    block.mlp.reset_parameters()
    assert all(float(p.detach().abs().sum()) > 0.0 for p in block.parameters())
    dense = Block(types.SimpleNamespace(hidden_size=16, intermediate_size=32))
    assert sorted(n for n, _ in dense.named_parameters()) == ["mlp.down_proj.weight", "mlp.gate_proj.weight", "mlp.up_proj.weight"]


def test_llama_module_tree_uses_the_reference_names():
    """picotron/model.py:363-402: ``embedding``, ``decoder_layers.N.{input_layernorm, post_attention_layernorm,
    attention.{q,k,v,out}_proj, mlp}``, ``final_proj``, ``final_norm``.  The reference's parameter counting keys on the
    substrings "attention", "mlp", "embed", "final_proj" (utils.py:88) besides the MoE ones; RoPE tables are plain
    attributes, not state (model.py:309-311)."""
    from picotron_amd.expert_parallel.expert_parallel import MoELayer
    from picotron_amd.model import MLP, Llama

    cfg = types.SimpleNamespace(vocab_size=50, hidden_size=16, intermediate_size=32, num_attention_heads=4,
                                num_key_value_heads=2, num_hidden_layers=2, max_position_embeddings=8, rms_norm_eps=1e-5,
                                rope_theta=10000.0, num_experts=4, num_experts_per_tok=2, num_shared_experts=1)
    model = Llama(cfg)
    names = [n for n, _ in model.named_parameters()]
    per_layer = ["input_layernorm.weight", "post_attention_layernorm.weight", "attention.q_proj.weight",
                 "attention.k_proj.weight", "attention.v_proj.weight", "attention.out_proj.weight", "mlp.gate.weight"]
    for i in range(2):
        for n in per_layer:
            assert f"decoder_layers.{i}.{n}" in names
        assert isinstance(model.decoder_layers[i].mlp, MoELayer)
    assert names[0] == "embedding.weight" and names[-2:] == ["final_proj.weight", "final_norm.weight"]
    assert model.decoder_layers[0].attention.k_proj.weight.shape == (8, 16)      # 2 kv heads x head_dim 4
    assert model.decoder_layers[0].cos.shape == (8, 4) and not any("cos" in k for k in model.state_dict())
    counted = [n for n in names if any(k in n.lower() for k in ("attention", "mlp", "embed", "final_proj"))]
    assert sorted(set(names) - set(counted)) == sorted(
        # "post_attention_layernorm" contains "attention", so the reference counts it with the split parameters
        [f"decoder_layers.{i}.input_layernorm.weight" for i in range(2)] + ["final_norm.weight"])
    cfg.parallel_block, cfg.num_experts = True, 1
    dense = Llama(cfg)
    assert isinstance(dense.decoder_layers[0].mlp, MLP) and not hasattr(dense.decoder_layers[0], "post_attention_layernorm")
    # embedding N(0,1), projections uniform in +-1/sqrt(fan_in) (model.py:147-155, 353-354)
    assert 0.8 < float(dense.embedding.weight.std()) < 1.2
    assert float(dense.final_proj.weight.abs().max()) <= 0.25


def test_cpu_tensors_are_refused_not_silently_computed():
    from picotron_amd.expert_parallel import megakernel
    from picotron_amd.expert_parallel.expert_parallel import MoELayer

    moe = MoELayer(_cfg())
    with pytest.raises(_lib.PicomoeError):
        moe(torch.randn(1, 4, 16))
    with pytest.raises(_lib.PicomoeError):
        megakernel.fused_moe(torch.randn(4, 16), torch.tensor([4]), torch.randn(1, 32, 16), torch.randn(1, 32, 16), torch.randn(1, 16, 32))
    if not torch.cuda.is_available():
        assert megakernel.cuda_available() is False


def test_combine_weights_follow_the_rows_dtype():
    """The combine kernels read gate weights and rows as one element type: the wrappers cast the weights to the rows'
    dtype (as the reference does, expert_parallel.py:184, capacity_moe.py:158) and refuse non-float or mis-sized ones
    before anything reaches a kernel."""
    from picotron_amd import _ops

    y = torch.zeros(6, 8, dtype=torch.bfloat16)
    w = torch.rand(3, 2, dtype=torch.float32)
    cast = _ops._weights_like(w, y)
    assert cast.dtype == torch.bfloat16 and cast.is_contiguous() and torch.equal(cast, w.bfloat16())
    assert _ops._weights_like(None, y) is None
    assert _ops._weights_like(w.bfloat16().t().contiguous().t(), y.float()).dtype == torch.float32
    with pytest.raises(_lib.PicomoeError):
        _ops._weights_like(torch.ones(3, 2, dtype=torch.int64), y)
    if os.path.exists(_lib.LIB_PATH):
        with pytest.raises(_lib.PicomoeError):  # 5 weights for 3 tokens x top-2: refused on the host
            _ops.combine_rows(y, torch.zeros(6, dtype=torch.int32), torch.rand(5), 3, 2)


def test_product_does_not_import_the_oracle():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dirpath, _, files in os.walk(os.path.join(root, "picotron_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower() or f == "README.md", os.path.join(dirpath, f)
