import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Two tiny configurations that differ in every size and option.
TINY_A = dict(architectures=["LlamaForCausalLM"], vocab_size=256, hidden_size=64, intermediate_size=176,
              num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=128, tie_word_embeddings=False,
              eos_token_id=2)
TINY_B = dict(architectures=["LlamaForCausalLM"], vocab_size=384, hidden_size=96, intermediate_size=256,
              num_hidden_layers=3, num_attention_heads=3, num_key_value_heads=1, head_dim=32,
              rms_norm_eps=1e-6, rope_theta=500000.0, max_position_embeddings=256, tie_word_embeddings=True,
              eos_token_id=7)
# A third one for sizes neither has: 5 query heads on 5 kv heads (no grouping), head_dim 48,
# a width and a vocabulary that are no power of two and no multiple of 64.
TINY_C = dict(architectures=["LlamaForCausalLM"], vocab_size=331, hidden_size=120, intermediate_size=200,
              num_hidden_layers=2, num_attention_heads=5, num_key_value_heads=5, head_dim=48,
              rms_norm_eps=1e-5, rope_theta=1000.0, max_position_embeddings=512, tie_word_embeddings=False,
              eos_token_id=1)
# A fourth with sizes the vector paths of the kernels do not like: a width and a feed-forward size that are no
# multiple of 8 (bfloat16 rows are then not 16-byte aligned), an odd vocabulary, heads wider than the width / heads.
TINY_D = dict(architectures=["LlamaForCausalLM"], vocab_size=301, hidden_size=70, intermediate_size=177,
              num_hidden_layers=2, num_attention_heads=3, num_key_value_heads=3, head_dim=32,
              rms_norm_eps=1e-4, rope_theta=5000.0, max_position_embeddings=160, tie_word_embeddings=True,
              eos_token_id=300)
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 5), "D": (TINY_D, 8)}


@pytest.fixture(scope="session")
def tiny_models(tmp_path_factory):
    """name -> (config dict, weights dict in float32, folder with float32 weights, folder with bfloat16 weights)."""
    from mini_inference_engine_amd.config import LlamaConfig
    from mini_inference_engine_amd.weights import random_tensors, write_random_model
    out = {}
    for name, (cfg, seed) in TINY.items():
        c = LlamaConfig.from_dict(cfg)
        f32 = str(tmp_path_factory.mktemp(f"tiny{name}_f32"))
        b16 = str(tmp_path_factory.mktemp(f"tiny{name}_bf16"))
        write_random_model(c, seed, f32, torch.float32)
        write_random_model(c, seed, b16, torch.bfloat16)
        out[name] = dict(cfg=cfg, config=c, seed=seed, weights=random_tensors(c, seed, torch.float32),
                         weights_bf16=random_tensors(c, seed, torch.bfloat16), folder_f32=f32, folder_bf16=b16)
    return out
