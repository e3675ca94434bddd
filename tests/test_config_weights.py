"""Configuration, registry, weight loading and the random-weights mode (no GPU)."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from conftest import TINY_A, TINY_B

from mini_inference_engine_amd.config import (ConfigError, EngineConfig, LlamaConfig, known_architectures,
                                              load_model_config, register_architecture, unregister_architecture)
from mini_inference_engine_amd.models import Decoder, build_llama
from mini_inference_engine_amd.weights import WeightError, load_weights, random_tensors, write_random_model


# ------------------------------------------------------------------ configuration
def test_llama_config_reads_its_own_keys_and_defaults():
    """Keys and defaults of inference_engine/config.py:26-42 there."""
    d = dict(vocab_size=100, hidden_size=48, intermediate_size=80, num_hidden_layers=2, num_attention_heads=3,
             rms_norm_eps=1e-6, max_position_embeddings=64)
    c = LlamaConfig.from_dict(d)
    assert c.num_key_value_heads == 3 and c.head_dim == 16 and c.rope_theta == 10000.0
    assert c.tie_word_embeddings is False and c.eos_token_id == (2,)
    c2 = LlamaConfig.from_dict({**d, "eos_token_id": [7, 9], "head_dim": 32, "num_key_value_heads": 1,
                                "rope_theta": 5e5, "tie_word_embeddings": True})
    assert (c2.eos_token_id, c2.head_dim, c2.num_key_value_heads, c2.rope_theta) == ((7, 9), 32, 1, 5e5)
    assert c2.to_dict()["eos_token_id"] == [7, 9] and c.to_dict()["eos_token_id"] == 2
    assert LlamaConfig.from_dict({**d, "head_dim": None}).head_dim == 16


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "rms_norm_eps", "max_position_embeddings"])
def test_required_keys(key):
    d = {k: v for k, v in TINY_A.items() if k != key}
    with pytest.raises(ConfigError, match=key):
        LlamaConfig.from_dict(d)


@pytest.mark.parametrize("bad, match", [
    ({"num_key_value_heads": 3}, "multiple"), ({"head_dim": 15}, "even"), ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "linear", "factor": 2}}, "rope_scaling"), ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"), ({"vocab_size": "many"}, "integer"), ({"rms_norm_eps": 0.0}, "positive"),
    ({"num_hidden_layers": 0}, ">= 1")])
def test_values_the_engine_does_not_compute_are_refused(bad, match):
    with pytest.raises(ConfigError, match=match):
        LlamaConfig.from_dict({**TINY_A, **bad})


def test_registry_chooses_by_name(tmp_path):
    assert "LlamaForCausalLM" in known_architectures()
    cfg, arch = load_model_config(TINY_A)
    assert arch.name == "LlamaForCausalLM" and isinstance(cfg, LlamaConfig)
    with pytest.raises(ConfigError, match="LlamaForCausalLM"):
        load_model_config({**TINY_A, "architectures": ["SomethingElse"]})
    no_arch = {k: v for k, v in TINY_A.items() if k != "architectures"}
    with pytest.raises(ConfigError, match="registered"):
        load_model_config(no_arch)
    assert load_model_config({**no_arch, "model_type": "llama"})[1].name == "LlamaForCausalLM"
    with open(tmp_path / "config.json", "w") as f:
        json.dump(TINY_B, f)
    assert load_model_config(str(tmp_path))[0].vocab_size == 384
    with pytest.raises(ConfigError, match="no config.json"):
        load_model_config(str(tmp_path / "nowhere"))


def test_another_architecture_registers_from_outside():
    class OtherConfig(LlamaConfig):
        architecture = "OtherForCausalLM"
    register_architecture("OtherForCausalLM", OtherConfig, build_llama)
    try:
        cfg, arch = load_model_config({**TINY_A, "architectures": ["OtherForCausalLM"]})
        assert type(cfg) is OtherConfig and arch.build is build_llama
        with pytest.raises(ValueError, match="already"):
            register_architecture("OtherForCausalLM", OtherConfig, build_llama)
    finally:
        unregister_architecture("OtherForCausalLM")
    assert "OtherForCausalLM" not in known_architectures()


def test_no_size_stands_in_code():
    """Every dimension of the assembled model follows the configuration: change each, see it move."""
    base = LlamaConfig.from_dict(TINY_A)
    shapes = {s.attr + "@" + s.sources[0].name: s.shape for _, s in Decoder(build_llama(base)).param_specs()}
    for key, value in [("vocab_size", 300), ("hidden_size", 80), ("intermediate_size", 100),
                       ("num_hidden_layers", 3), ("num_attention_heads", 8), ("num_key_value_heads", 1),
                       ("head_dim", 32)]:
        other = LlamaConfig.from_dict({**TINY_A, key: value})
        moved = {s.attr + "@" + s.sources[0].name: s.shape for _, s in Decoder(build_llama(other)).param_specs()}
        assert moved != shapes, f"{key} changes nothing"
    layer = build_llama(LlamaConfig.from_dict({**TINY_A, "rms_norm_eps": 3e-3, "rope_theta": 77.0})).layers[0]
    assert layer.norm_mixer.eps == 3e-3 and layer.mixer.position.theta == 77.0
    assert layer.mixer.scale == 16 ** -0.5


def test_engine_config_validation():
    with pytest.raises(ValueError):
        EngineConfig(block_size=24)
    with pytest.raises(ValueError):
        EngineConfig(num_blocks=1)
    with pytest.raises(ValueError, match="unknown"):
        EngineConfig.with_overrides(None, no_such_knob=1)
    assert EngineConfig.with_overrides(EngineConfig(block_size=32), max_num_seqs=4).block_size == 32


# ------------------------------------------------------------------------ weights
def build(cfg_dict):
    return Decoder(build_llama(LlamaConfig.from_dict(cfg_dict)))


def test_random_model_folder_round_trip(tmp_path):
    cfg = LlamaConfig.from_dict(TINY_B)
    folder = write_random_model(cfg, 1, str(tmp_path / "m"), torch.bfloat16)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    again, _ = load_model_config(folder)
    assert again == cfg
    stored = load_file(os.path.join(folder, "model.safetensors"))
    assert all(t.dtype == torch.bfloat16 for t in stored.values())
    assert "lm_head.weight" not in stored, "tied embeddings: no separate head is written"
    assert torch.equal(stored["model.norm.weight"], random_tensors(cfg, 1, torch.bfloat16)["model.norm.weight"])
    assert not torch.equal(stored["model.norm.weight"], random_tensors(cfg, 2, torch.bfloat16)["model.norm.weight"])
    w = random_tensors(cfg, 1, torch.float32)
    assert abs(float(w["model.embed_tokens.weight"].std()) - 0.02) < 2e-3
    assert abs(float(w["model.norm.weight"].mean()) - 1.0) < 1e-2


def test_loader_fuses_by_name_and_keeps_dtypes(tmp_path):
    cfg = LlamaConfig.from_dict(TINY_A)
    w = random_tensors(cfg, 0, torch.bfloat16)
    w["model.norm.weight"] = w["model.norm.weight"].float()          # a tensor stored in 32-bit stays so
    model = build(TINY_A)
    load_weights(model, w, "cpu", torch.bfloat16)
    att = model.spec.layers[1].mixer
    p = "model.layers.1.self_attn."
    assert torch.equal(att.w_qkv, torch.cat([w[p + "q_proj.weight"], w[p + "k_proj.weight"], w[p + "v_proj.weight"]]))
    ff = model.spec.layers[0].feed_forward
    assert torch.equal(ff.w_gate_up[:176], w["model.layers.0.mlp.gate_proj.weight"])
    assert torch.equal(ff.w_gate_up[176:], w["model.layers.0.mlp.up_proj.weight"])
    assert att.w_qkv.dtype == torch.bfloat16 and model.spec.final_norm.weight.dtype == torch.float32
    model32 = build(TINY_A)
    load_weights(model32, w, "cpu", torch.float32)
    assert all(getattr(p_, s.attr).dtype == torch.float32 for p_, s in model32.param_specs())
    assert torch.equal(model32.spec.layers[1].mixer.w_o, w[p + "o_proj.weight"].float())


def test_tied_and_untied_heads():
    tied = build(TINY_B)
    w = random_tensors(LlamaConfig.from_dict(TINY_B), 1, torch.float32)
    load_weights(tied, {**w, "lm_head.weight": torch.zeros(384, 96)}, "cpu", torch.float32)   # ignored, not an error
    assert tied.spec.head.weight is tied.spec.embedding.weight
    untied = build(TINY_A)
    wa = random_tensors(LlamaConfig.from_dict(TINY_A), 0, torch.float32)
    load_weights(untied, wa, "cpu", torch.float32)
    assert untied.spec.head.weight is not untied.spec.embedding.weight
    assert torch.equal(untied.spec.head.weight, wa["lm_head.weight"])


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = LlamaConfig.from_dict(TINY_A)
    w = random_tensors(cfg, 0, torch.float32)
    del w["model.layers.0.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.7.mlp.up_proj.weight"] = torch.zeros(2, 2)
    w["model.layers.1.self_attn.k_proj.weight"] = torch.zeros(16, 64)
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)       # known leftover: skipped
    save_file(w, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        load_weights(build(TINY_A), str(tmp_path), "cpu", torch.float32)
    err = e.value
    assert err.missing == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.mlp.up_proj.weight"]
    assert [(n, tuple(f), tuple(x)) for n, f, x in err.wrong_shape] == \
        [("model.layers.1.self_attn.k_proj.weight", (16, 64), (32, 64))]
    text = str(err)
    for needle in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (1)", "expected (32, 64)"):
        assert needle in text


def test_no_safetensors_and_sharded_folders(tmp_path):
    with pytest.raises(FileNotFoundError, match="no .safetensors"):
        load_weights(build(TINY_A), str(tmp_path), "cpu", torch.float32)
    w = random_tensors(LlamaConfig.from_dict(TINY_A), 0, torch.float32)
    names = sorted(w)
    half = len(names) // 2
    save_file({n: w[n] for n in names[:half]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({n: w[n] for n in names[half:]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    index = {"weight_map": {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                            for i, n in enumerate(names)}}
    with open(tmp_path / "model.safetensors.index.json", "w") as f:
        json.dump(index, f)
    model = build(TINY_A)
    load_weights(model, str(tmp_path), "cpu", torch.float32)
    assert torch.equal(model.spec.embedding.weight, w["model.embed_tokens.weight"])


def test_float32_matrices_in_bfloat16_mode_are_reported(tiny_models):
    """A tensor stored in 32-bit stays so; for a matrix that means the slow 32-bit products, so the load
    report names it (and the entry point warns)."""
    from mini_inference_engine_amd.models.decoder import Decoder
    from mini_inference_engine_amd.config.registry import architecture_of
    from mini_inference_engine_amd.weights import load_weights
    m = tiny_models["A"]
    mixed = dict(m["weights_bf16"])
    mixed["model.layers.1.mlp.down_proj.weight"] = m["weights"]["model.layers.1.mlp.down_proj.weight"]      # float32
    mixed["model.norm.weight"] = m["weights"]["model.norm.weight"]                                          # a vector
    model = Decoder(architecture_of(m["config"]).build(m["config"]))
    report = load_weights(model, mixed, "cpu", torch.bfloat16)
    assert report["kept_float32"] == ["model.layers.1.mlp.down_proj.weight"], "matrices only; vectors are cheap"
    assert model.spec.layers[1].feed_forward.w_down.dtype == torch.float32
    assert model.spec.layers[0].feed_forward.w_down.dtype == torch.bfloat16
    report = load_weights(Decoder(architecture_of(m["config"]).build(m["config"])), m["weights_bf16"], "cpu", torch.bfloat16)
    assert report["kept_float32"] == []


# ------------------------------------------------------------------ a checkpoint that stores things differently
def test_checkpoint_with_fused_transposed_and_interleaved_tensors(tmp_path):
    """A toy architecture registered here, Llama's layers with another checkpoint layout: one fused q/k/v
    tensor stored [in, out] (each projection is a range of its columns, transposed), gate and up rows
    interleaved in one tensor (a transform registered here takes them apart), and an integer table (a token
    remapping) in front of the embedding.  Its parts only declare where their rows come from; the loader and
    the random-weights mode are not touched.  The same numbers rearranged into Llama's layout must give Llama's
    logits, bit for bit, through the real runner."""
    from dataclasses import dataclass
    import numpy as np
    from torch_backend import TorchBackend
    from mini_inference_engine_amd.config import ModelConfig, register_architecture, unregister_architecture
    from mini_inference_engine_amd.engine.batch import StepRow
    from mini_inference_engine_amd.engine.runner import ModelRunner
    from mini_inference_engine_amd.parts import (Attention, DecoderSpec, Embedding, LMHead, ParamSpec, PreNormBlock, RMSNorm,
                                                 RotaryHalfSplit, Source, SwiGLU, register_weight_transform)
    from mini_inference_engine_amd.weights import write_random_model
    base = LlamaConfig.from_dict(TINY_A)
    h, H, Hkv, D, I, V = (base.hidden_size, base.num_attention_heads, base.num_key_value_heads, base.head_dim,
                          base.intermediate_size, base.vocab_size)
    register_weight_transform("even_rows", lambda t: t[0::2])
    register_weight_transform("odd_rows", lambda t: t[1::2])

    class PackedAttention(Attention):
        def params(self):
            p, n = self.prefix, (H + 2 * Hkv) * D
            def cols(a, b):
                return Source(f"{p}.qkv_packed", (b - a, h), stored_shape=(h, n), cols=(a, b), transform="transpose")
            return [ParamSpec.stacked("w_qkv", [cols(0, H * D), cols(H * D, (H + Hkv) * D), cols((H + Hkv) * D, n)]),
                    ParamSpec.single("w_o", f"{p}.o_proj.weight", (h, H * D))]

    class InterleavedSwiGLU(SwiGLU):
        def params(self):
            p = self.prefix
            return [ParamSpec.stacked("w_gate_up", [
                        Source(f"{p}.gate_up_interleaved", (I, h), stored_shape=(2 * I, h), transform="even_rows"),
                        Source(f"{p}.gate_up_interleaved", (I, h), stored_shape=(2 * I, h), transform="odd_rows")]),
                    ParamSpec.single("w_down", f"{p}.down_proj.weight", (h, I))]

    class RemappedEmbedding(Embedding):
        remap = None

        def params(self):
            return super().params() + [ParamSpec.single("remap", "token_remap", (V,), integer=True, integer_bound=V)]

        def forward(self, ids, taken_from=None, earlier_tokens=None):
            return self.ops.embedding(self.remap[ids.long()], self.weight, taken_from, earlier_tokens)

    @dataclass(frozen=True)
    class PackedConfig(ModelConfig):
        layers: int = base.num_hidden_layers
        architecture = "PackedToyForCausalLM"

        def to_dict(self):
            return {"architectures": [self.architecture], "layers": self.layers}

        @classmethod
        def from_dict(cls, d):
            return cls(layers=d["layers"])

    def build_packed(cfg):
        rope = RotaryHalfSplit(D, base.rope_theta, base.max_position_embeddings)
        layers = [PreNormBlock(RMSNorm(h, base.rms_norm_eps, f"l{i}.n1"),
                               PackedAttention(h, H, Hkv, D, scale=D ** -0.5, position=rope, prefix=f"l{i}.att"),
                               RMSNorm(h, base.rms_norm_eps, f"l{i}.n2"), InterleavedSwiGLU(h, I, f"l{i}.ff"))
                  for i in range(cfg.layers)]
        emb = RemappedEmbedding(V, h, "emb")
        return DecoderSpec(embedding=emb, layers=layers, final_norm=RMSNorm(h, base.rms_norm_eps, "out_norm"),
                           head=LMHead(V, h, "head"), max_position=base.max_position_embeddings, vocab_size=V)

    register_architecture("PackedToyForCausalLM", PackedConfig, build_packed, shapes={"packed-toy": {"layers": 2}},
                          replace=True)
    try:
        from mini_inference_engine_amd.config import known_shapes, shape_config
        assert "packed-toy" in known_shapes() and shape_config("packed-toy") == PackedConfig(2)
        folder = write_random_model(PackedConfig(), 4, str(tmp_path / "packed"), torch.float32)
        from safetensors.torch import load_file
        stored = load_file(f"{folder}/model.safetensors")
        assert tuple(stored["l0.att.qkv_packed"].shape) == (h, (H + 2 * Hkv) * D)
        assert tuple(stored["l1.ff.gate_up_interleaved"].shape) == (2 * I, h)
        remap = stored["token_remap"]
        assert remap.dtype == torch.int32 and int(remap.min()) >= 0 and int(remap.max()) < V and len(set(remap.tolist())) > V // 4
        runner = ModelRunner(folder, dtype="float32", device="cpu", backend=TorchBackend(torch.float32), num_pages=8,
                             max_rows=2, max_step_tokens=64)
        att, ff = runner.model.spec.layers[1].mixer, runner.model.spec.layers[1].feed_forward
        assert torch.equal(att.w_qkv, stored["l1.att.qkv_packed"].t()) and att.w_qkv.is_contiguous()
        assert torch.equal(ff.w_gate_up[:I], stored["l1.ff.gate_up_interleaved"][0::2])
        assert torch.equal(ff.w_gate_up[I:], stored["l1.ff.gate_up_interleaved"][1::2])
        assert runner.model.spec.embedding.remap.dtype == torch.int32
        # the same numbers in Llama's layout
        llama = {"model.embed_tokens.weight": stored["emb"][remap.long()], "lm_head.weight": stored["head"],
                 "model.norm.weight": stored["out_norm"]}
        for i in range(2):
            q, k, v = stored[f"l{i}.att.qkv_packed"].t().split([H * D, Hkv * D, Hkv * D])
            p = f"model.layers.{i}."
            llama.update({p + "self_attn.q_proj.weight": q.contiguous(), p + "self_attn.k_proj.weight": k.contiguous(),
                          p + "self_attn.v_proj.weight": v.contiguous(), p + "self_attn.o_proj.weight": stored[f"l{i}.att.o_proj.weight"],
                          p + "mlp.gate_proj.weight": stored[f"l{i}.ff.gate_up_interleaved"][0::2].contiguous(),
                          p + "mlp.up_proj.weight": stored[f"l{i}.ff.gate_up_interleaved"][1::2].contiguous(),
                          p + "mlp.down_proj.weight": stored[f"l{i}.ff.down_proj.weight"],
                          p + "input_layernorm.weight": stored[f"l{i}.n1"], p + "post_attention_layernorm.weight": stored[f"l{i}.n2"]})
        as_llama = ModelRunner(base, weights=llama, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                               num_pages=8, max_rows=2, max_step_tokens=64)
        toks = torch.randint(0, V, (37,), generator=torch.Generator().manual_seed(1)).tolist()
        outs = []
        for r in (runner, as_llama):
            rc = r.cache.open("a")
            assert r.cache.reserve(rc, 0, len(toks))
            outs.append(r.forward_step([StepRow(rc, toks, 0, list(range(len(toks))))]))
        assert torch.equal(outs[0], outs[1])
        # a checkpoint whose fused tensor has another shape is reported with the stored shape, once
        bad = dict(stored)
        bad["l0.att.qkv_packed"] = torch.zeros(h, 5)
        with pytest.raises(WeightError) as e:
            ModelRunner(PackedConfig(), weights=bad, dtype="float32", device="cpu", backend=TorchBackend(torch.float32),
                        num_pages=8)
        assert [(n, tuple(f), tuple(x)) for n, f, x in e.value.wrong_shape] == [("l0.att.qkv_packed", (h, 5), (h, (H + 2 * Hkv) * D))]
    finally:
        unregister_architecture("PackedToyForCausalLM")
