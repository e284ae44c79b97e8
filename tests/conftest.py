import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:  # noqa: BLE001
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU is visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# ---- the two tiny configurations: they differ in every size and option ----------
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 172, "vocab_size": 256, "max_position_embeddings": 128,
    "rope_theta": 10000.0, "rope_scaling": None, "rms_norm_eps": 1e-5, "tie_word_embeddings": True,
    "hidden_act": "silu",
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 256, "vocab_size": 320, "max_position_embeddings": 256,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "hidden_act": "silu",
}
# a third one with room for long sequences: head size 48 (not a power of two), 5 heads on 5 KV heads
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 80, "num_attention_heads": 6, "num_key_value_heads": 3,
    "head_dim": 48, "intermediate_size": 200, "vocab_size": 500, "max_position_embeddings": 2048,
    "rope_theta": 10000.0, "rope_scaling": None, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
    "hidden_act": "silu",
}
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C}


def make_model_folder(path, config_json, seed, dtype="float32", std=0.02, norm_init=None, device="cpu"):
    import torch
    import hfee_amd  # noqa: F401  (registers the architecture)
    from hfee_amd.config import config_from_dict
    from hfee_amd.weights import write_model_folder
    cfg = config_from_dict(config_json)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    return write_model_folder(str(path), cfg, seed=seed, std=std, dtype=dt, norm_init=norm_init, device=device)


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name -> folder, for the tiny configurations in both storage types.  Weights have
    std 0.1 so that attention and logits are far from uniform."""
    out = {}
    base = tmp_path_factory.mktemp("models")
    for name, cj in TINY.items():
        for dtype in ("float32", "bfloat16"):
            out[(name, dtype)] = make_model_folder(base / f"{name}_{dtype}", cj, seed=11 + ord(name),
                                                   dtype=dtype, std=0.1,
                                                   norm_init="one_plus_normal" if name != "B" else "normal")
    return out
