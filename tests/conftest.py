"""Shared fixtures: two tiny Qwen2-MoE configurations that differ in every
size and option, model folders with seeded random weights made in temporary
folders, and the `gpu` marker."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


CONFIG_A = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 128,
    "moe_intermediate_size": 32, "shared_expert_intermediate_size": 64,
    "num_experts": 4, "num_experts_per_tok": 2, "norm_topk_prob": False,
    "decoder_sparse_step": 1, "mlp_only_layers": [], "vocab_size": 256,
    "rope_theta": 10000.0, "use_sliding_window": False, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "hidden_act": "silu",
}

CONFIG_B = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3,
    "num_key_value_heads": 1, "head_dim": 32, "intermediate_size": 192,
    "moe_intermediate_size": 48, "shared_expert_intermediate_size": 80,
    "num_experts": 8, "num_experts_per_tok": 3, "norm_topk_prob": True,
    "decoder_sparse_step": 2, "mlp_only_layers": [0], "vocab_size": 384,
    "rope_theta": 1000000.0, "use_sliding_window": True, "sliding_window": 24,
    "max_window_layers": 2, "rms_norm_eps": 1e-5, "tie_word_embeddings": True,
    "hidden_act": "gelu_pytorch_tanh",
}

# Heads of 64 in groups of three, so that the engine's bf16 steps run the matrix-core
# attention kernels (prompt portions, and decoding with grouped heads); one layer sees all
# keys, one a window.
CONFIG_C = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "num_hidden_layers": 2, "hidden_size": 128, "num_attention_heads": 6,
    "num_key_value_heads": 2, "head_dim": 64, "intermediate_size": 160,
    "moe_intermediate_size": 64, "shared_expert_intermediate_size": 96,
    "num_experts": 6, "num_experts_per_tok": 2, "norm_topk_prob": True,
    "decoder_sparse_step": 1, "mlp_only_layers": [], "vocab_size": 320,
    "rope_theta": 500000.0, "use_sliding_window": True, "sliding_window": 40,
    "max_window_layers": 1, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
    "hidden_act": "silu",
}

TINY = {"A": (CONFIG_A, 1234), "B": (CONFIG_B, 987), "C": (CONFIG_C, 4321)}
# Std of the random weights. With tiny widths, N(0, 0.02) leaves all logits and attention
# scores near zero, which would hide faults: 0.1. C is wider, and 0.08 keeps its logits at
# the size (std about 0.9) that the bf16 bounds of the tests were made for.
TINY_STD = {"A": 0.1, "B": 0.1, "C": 0.08}


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """name -> dtype -> folder with config.json and model.safetensors."""
    import ninfer_amd
    out = {}
    for name, (cfg, seed) in TINY.items():
        out[name] = {}
        for dtype in ("float32", "bfloat16"):
            d = str(tmp_path_factory.mktemp(f"tiny_{name}_{dtype}"))
            ninfer_amd.write_random_model(d, cfg, seed, dtype=dtype, std=TINY_STD[name])
            out[name][dtype] = d
    return out
