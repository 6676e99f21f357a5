"""Configuration, registry, weight reading and its errors (CPU)."""
import json
import os
import struct

import pytest
import torch

import util
from conftest import CONFIG_A, CONFIG_B


def test_typed_configuration_of_both_tiny_models():
    from ninfer_amd import Qwen2MoeConfig
    a, b = Qwen2MoeConfig.from_dict(CONFIG_A), Qwen2MoeConfig.from_dict(CONFIG_B)
    assert (a.num_hidden_layers, a.hidden_size, a.head_dim, a.num_key_value_heads) == (2, 64, 16, 2)
    assert [a.layer_is_sparse(l) for l in range(2)] == [True, True]
    assert [b.layer_is_sparse(l) for l in range(3)] == [False, True, False]
    assert [b.layer_window(l) for l in range(3)] == [None, None, 24]
    assert b.tie_word_embeddings and b.norm_topk_prob and b.rms_norm_eps == 1e-5
    assert a.rope_theta == 10000.0 and b.rope_theta == 1e6


def test_defaults_follow_the_reference():
    from ninfer_amd import Qwen2MoeConfig
    raw = {k: v for k, v in CONFIG_A.items()
           if k not in ("num_key_value_heads", "head_dim", "rope_theta", "tie_word_embeddings",
                        "norm_topk_prob", "decoder_sparse_step", "mlp_only_layers")}
    c = Qwen2MoeConfig.from_dict(raw)
    assert c.num_key_value_heads == c.num_attention_heads == 4      # config.cpp:21-23
    assert c.head_dim == 64 // 4                                     # config.cpp:25-27
    assert c.rope_theta == 1e6 and c.tie_word_embeddings is False    # config.cpp:29-32
    assert c.decoder_sparse_step == 1 and c.mlp_only_layers == [] and c.norm_topk_prob is False


@pytest.mark.parametrize("change,word", [
    ({"vocab_size": None}, "vocab_size"), ({"rms_norm_eps": None}, "rms_norm_eps"),
    ({"num_experts": -1}, "num_experts"), ({"hidden_size": "64"}, "hidden_size"),
    ({"moe_intermediate_size": None}, "moe_intermediate_size"), ({"eos_token_id": [3, "x"]}, "eos_token_id"),
    ({"num_key_value_heads": 3}, "num_key_value_heads"), ({"num_experts_per_tok": 9}, "num_experts_per_tok"),
    ({"hidden_act": "gelu"}, "hidden_act"), ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
    ({"model_type": "llama"}, "model_type"), ({"use_sliding_window": True}, "sliding_window"),
    ({"mlp_only_layers": [5]}, "mlp_only_layers"), ({"head_dim": 15}, "head_dim"),
    ({"shared_expert_intermediate_size": -2}, "shared_expert_intermediate_size"),
    ({"num_hidden_layers": 0}, "num_hidden_layers"), ({"tie_word_embeddings": "yes"}, "tie_word_embeddings"),
])
def test_configuration_errors_name_the_key(change, word):
    from ninfer_amd import ConfigError, Qwen2MoeConfig
    raw = dict(CONFIG_A)
    for k, v in change.items():
        if v is None:
            raw.pop(k)
        else:
            raw[k] = v
    with pytest.raises(ConfigError, match=word):
        Qwen2MoeConfig.from_dict(raw)


def test_rope_keys_and_qkv_bias():
    """The rotation's base may stand inside 'rope_parameters'; scaling of the plain kind is
    no scaling; another kind is refused. Without `qkv_bias` the model asks for no biases."""
    from ninfer_amd import ConfigError, Qwen2MoeConfig
    from ninfer_amd.loading import build_spec
    raw = dict(CONFIG_A)
    del raw["rope_theta"]
    raw["rope_parameters"] = {"rope_type": "default", "rope_theta": 12345.0}
    assert Qwen2MoeConfig.from_dict(raw).rope_theta == 12345.0
    raw = dict(CONFIG_A, rope_scaling={"type": "default"})
    assert Qwen2MoeConfig.from_dict(raw).rope_theta == CONFIG_A["rope_theta"]
    with pytest.raises(ConfigError, match="rope_parameters"):
        Qwen2MoeConfig.from_dict(dict(CONFIG_A, rope_parameters={"rope_type": "linear", "factor": 2.0}))
    with pytest.raises(ConfigError, match="qkv_bias"):
        Qwen2MoeConfig.from_dict(dict(CONFIG_A, qkv_bias=1))
    assert Qwen2MoeConfig.from_dict(CONFIG_A).qkv_bias is True
    _, with_bias = build_spec(CONFIG_A)
    _, without = build_spec(dict(CONFIG_A, qkv_bias=False))
    dropped = set(with_bias.tensor_specs()) - set(without.tensor_specs())
    assert len(dropped) == 3 * CONFIG_A["num_hidden_layers"]
    assert all(n.endswith("_proj.bias") for n in dropped)


def test_keys_that_may_be_absent_or_lists():
    """`eos_token_id` is one id or a list, and every id of the list ends a generation; without
    experts every layer is dense and asks for no expert tensors; without a shared expert a
    sparse layer has none of its tensors."""
    from ninfer_amd import Qwen2MoeConfig
    from ninfer_amd.loading import build_spec
    from ninfer_amd.parts import SparseMoE, SwiGLU
    assert Qwen2MoeConfig.from_dict(CONFIG_A).eos_token_ids == ()
    assert Qwen2MoeConfig.from_dict(dict(CONFIG_A, eos_token_id=7)).eos_token_ids == (7,)
    c = Qwen2MoeConfig.from_dict(dict(CONFIG_A, eos_token_id=[9, 4]))
    assert c.eos_token_ids == (9, 4) and c.eos_token_id == 9
    _, spec = build_spec(dict(CONFIG_A, eos_token_id=[9, 4]))
    assert spec.eos_token_ids == (9, 4)
    dense = {k: v for k, v in CONFIG_A.items() if k not in (
        "num_experts", "num_experts_per_tok", "moe_intermediate_size",
        "shared_expert_intermediate_size")}
    cfg, spec = build_spec(dense)
    assert cfg.num_experts == 0 and all(type(b.feed_forward) is SwiGLU for b in spec.blocks)
    assert not any("expert" in n or ".gate.weight" in n for n in spec.tensor_specs())
    no_shared = {k: v for k, v in CONFIG_A.items() if k != "shared_expert_intermediate_size"}
    _, spec = build_spec(no_shared)
    assert all(type(b.feed_forward) is SparseMoE and b.feed_forward.shared is None
               for b in spec.blocks)
    assert not any("shared_expert" in n for n in spec.tensor_specs())
    assert "model.layers.0.mlp.experts.3.up_proj.weight" in spec.tensor_specs()


def test_registry_resolves_by_architecture_name():
    import ninfer_amd
    from ninfer_amd.loading import build_spec
    assert "Qwen2MoeForCausalLM" in ninfer_amd.architectures()
    with pytest.raises(KeyError, match="registered: .*Qwen2MoeForCausalLM"):
        build_spec(dict(CONFIG_A, architectures=["NoSuchModel"]))
    with pytest.raises(ninfer_amd.ConfigError, match="architectures"):
        build_spec({k: v for k, v in CONFIG_A.items() if k != "architectures"})


def test_layer_kinds_and_tensor_names_follow_the_configuration():
    from ninfer_amd.loading import build_spec
    from ninfer_amd.parts import SparseMoE, SwiGLU
    _, spec = build_spec(CONFIG_B)
    kinds = [type(b.feed_forward) for b in spec.blocks]
    assert kinds == [SwiGLU, SparseMoE, SwiGLU]
    assert [b.mixer.window for b in spec.blocks] == [None, None, 24]
    names = spec.tensor_specs()
    assert "lm_head.weight" not in names                     # tied
    assert names["model.layers.0.mlp.gate_proj.weight"].shape == (192, 96)
    assert names["model.layers.1.mlp.experts.7.down_proj.weight"].shape == (96, 48)
    assert names["model.layers.1.mlp.shared_expert_gate.weight"].shape == (1, 96)
    assert names["model.layers.1.mlp.gate.weight"].shape == (8, 96)
    assert "model.layers.1.mlp.gate_proj.weight" not in names
    assert names["model.layers.2.self_attn.k_proj.bias"].shape == (32,)
    assert "model.layers.2.self_attn.o_proj.bias" not in names
    _, spec_a = build_spec(CONFIG_A)
    assert "lm_head.weight" in spec_a.tensor_specs()


def test_random_folder_round_trip(model_dirs):
    """What the random-weights mode wrote is what the engine's reader returns,
    tensor by tensor, and what an independent reader (safetensors) sees."""
    from ninfer_amd.weights import CheckpointSource
    for dtype, torch_dtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        d = model_dirs["B"][dtype]
        _, ref = util.read_folder(d)
        src = CheckpointSource(d)
        assert set(src.shapes()) == set(ref)
        for name, t in ref.items():
            got = src.read(name)
            assert got.dtype == torch_dtype, "bfloat16 stays bfloat16, 32-bit stays 32-bit"
            assert torch.equal(got.float(), t)
        gains = ref["model.norm.weight"]
        assert abs(float(gains.mean()) - 1.0) < 0.1            # gains are 1 + noise
        assert abs(float(ref["model.layers.0.self_attn.q_proj.weight"].mean())) < 0.02
        src.close()


def test_same_seed_same_weights_other_seed_other_weights(tmp_path):
    import ninfer_amd
    for name, seed in (("a", 1), ("b", 1), ("c", 2)):
        ninfer_amd.write_random_model(str(tmp_path / name), CONFIG_A, seed)
    ta = util.read_folder(str(tmp_path / "a"))[1]
    tb = util.read_folder(str(tmp_path / "b"))[1]
    tc = util.read_folder(str(tmp_path / "c"))[1]
    assert all(torch.equal(ta[k], tb[k]) for k in ta)
    assert not torch.equal(ta["lm_head.weight"], tc["lm_head.weight"])


def _rewrite(src_dir, dst_dir, edit):
    """Copy a model folder, editing the name -> tensor dictionary."""
    from ninfer_amd.weights import write_safetensors
    cfg, tensors = util.read_folder(src_dir)
    edit(tensors)
    os.makedirs(dst_dir, exist_ok=True)
    with open(os.path.join(dst_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(dst_dir, "model.safetensors"), sorted(tensors.items()))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(model_dirs, tmp_path):
    from ninfer_amd.loading import build_spec
    from ninfer_amd.weights import CheckpointSource, WeightError, check_tensors

    def edit(t):
        del t["model.layers.0.self_attn.q_proj.bias"]
        del t["model.layers.1.mlp.experts.2.up_proj.weight"]
        t["model.layers.0.extra.weight"] = torch.zeros(3)
        t["model.norm.weight"] = torch.zeros(65)
        t["model.layers.1.mlp.gate.weight"] = torch.zeros(64, 4)

    d = str(tmp_path / "broken")
    _rewrite(model_dirs["A"]["float32"], d, edit)
    cfg, spec = build_spec(CONFIG_A)
    with pytest.raises(WeightError) as e:
        check_tensors(CheckpointSource(d).shapes(), spec.tensor_specs(), d)
    msg = str(e.value)
    assert "missing tensors (2)" in msg and "model.layers.0.self_attn.q_proj.bias" in msg
    assert "model.layers.1.mlp.experts.2.up_proj.weight" in msg
    assert "unexpected tensors (1)" in msg and "model.layers.0.extra.weight" in msg
    assert "wrong shapes (2)" in msg and "has [65], expected [64]" in msg
    assert "has [64, 4], expected [4, 64]" in msg


def test_tensors_a_checkpoint_may_hold_unread(model_dirs, tmp_path):
    """A tied model's checkpoint may carry a copy of the head, an older one the rotation's
    frequency tables: passed over when their shapes are right, reported when not."""
    from ninfer_amd.loading import build_spec
    from ninfer_amd.weights import CheckpointSource, WeightError, check_tensors
    cfg, spec = build_spec(CONFIG_B)
    half = CONFIG_B["head_dim"] // 2

    def edit(t):
        t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
        t["model.layers.1.self_attn.rotary_emb.inv_freq"] = torch.zeros(half)

    d = str(tmp_path / "extra")
    _rewrite(model_dirs["B"]["float32"], d, edit)
    check_tensors(CheckpointSource(d).shapes(), spec.tensor_specs(), d, spec.unused_tensor_specs())
    with pytest.raises(WeightError, match="unexpected tensors \\(2\\)"):
        check_tensors(CheckpointSource(d).shapes(), spec.tensor_specs(), d)

    def edit_wrong(t):
        t["lm_head.weight"] = torch.zeros(3, CONFIG_B["hidden_size"])

    d2 = str(tmp_path / "extra_wrong")
    _rewrite(model_dirs["B"]["float32"], d2, edit_wrong)
    with pytest.raises(WeightError, match="wrong shapes \\(1\\)"):
        check_tensors(CheckpointSource(d2).shapes(), spec.tensor_specs(), d2,
                      spec.unused_tensor_specs())
    # an untied model reads its head: nothing of it is passed over
    _, untied = build_spec(CONFIG_A)
    assert "lm_head.weight" in untied.tensor_specs()
    assert "lm_head.weight" not in untied.unused_tensor_specs()


def test_file_level_errors(tmp_path):
    from ninfer_amd.weights import SafeTensorsFile, WeightError
    with pytest.raises(WeightError, match="no such file"):
        SafeTensorsFile(str(tmp_path / "nope.safetensors"))
    p = tmp_path / "short.safetensors"
    p.write_bytes(b"abc")
    with pytest.raises(WeightError, match="too short"):
        SafeTensorsFile(str(p))
    p = tmp_path / "len.safetensors"
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(WeightError, match="header length"):
        SafeTensorsFile(str(p))
    p = tmp_path / "json.safetensors"
    p.write_bytes(struct.pack("<Q", 4) + b"{{{{")
    with pytest.raises(WeightError, match="not valid JSON"):
        SafeTensorsFile(str(p))

    def with_header(h, payload=b""):
        raw = json.dumps(h).encode()
        q = tmp_path / "h.safetensors"
        q.write_bytes(struct.pack("<Q", len(raw)) + raw + payload)
        return str(q)

    with pytest.raises(WeightError, match="malformed"):
        SafeTensorsFile(with_header({"x": {"dtype": "F32", "shape": [2]}}))
    with pytest.raises(WeightError, match="unsupported dtype"):
        SafeTensorsFile(with_header({"x": {"dtype": "F8_E4M3", "shape": [2], "data_offsets": [0, 2]}},
                                    b"ab"))
    with pytest.raises(WeightError, match="spans bytes"):
        SafeTensorsFile(with_header({"x": {"dtype": "F32", "shape": [2], "data_offsets": [0, 4]}},
                                    b"abcd"))
    f = SafeTensorsFile(with_header({"__metadata__": {"format": "pt"},
                                     "x": {"dtype": "F16", "shape": [2], "data_offsets": [0, 4]},
                                     "i": {"dtype": "I64", "shape": [1], "data_offsets": [4, 12]}},
                                    torch.tensor([1.5, -2.0], dtype=torch.float16).numpy().tobytes()
                                    + struct.pack("<q", 7)))
    assert set(f.tensors) == {"x", "i"}


def test_kept_dtypes_and_missing_name(tmp_path):
    from ninfer_amd.weights import CheckpointSource, WeightError, write_safetensors
    d = tmp_path / "m"
    d.mkdir()
    write_safetensors(str(d / "model.safetensors"),
                      [("h", torch.tensor([1.5, 2.5], dtype=torch.float16)),
                       ("b", torch.tensor([1.0, 3.0], dtype=torch.bfloat16)),
                       ("f", torch.tensor([0.1], dtype=torch.float32)),
                       ("table", torch.tensor([3, 4], dtype=torch.int64))])
    src = CheckpointSource(str(d))
    assert src.read("h").dtype == torch.float32 and src.read("b").dtype == torch.bfloat16
    assert src.read("f").dtype == torch.float32 and src.read("table").dtype == torch.int32
    assert src.read("table").tolist() == [3, 4]
    with pytest.raises(WeightError, match="missing tensor in checkpoint: nope"):
        src.read("nope")


def test_sharded_folder_with_index(model_dirs, tmp_path):
    from ninfer_amd.weights import CheckpointSource, write_safetensors
    cfg, tensors = util.read_folder(model_dirs["A"]["float32"])
    names = sorted(tensors)
    half = len(names) // 2
    shards = {"model-00001-of-00002.safetensors": names[:half],
              "model-00002-of-00002.safetensors": names[half:]}
    weight_map = {}
    for fn, ns in shards.items():
        write_safetensors(str(tmp_path / fn), [(n, tensors[n]) for n in ns])
        weight_map.update({n: fn for n in ns})
    with open(tmp_path / "model.safetensors.index.json", "w") as f:
        json.dump({"weight_map": weight_map}, f)
    src = CheckpointSource(str(tmp_path))
    assert set(src.shapes()) == set(names)
    assert torch.equal(src.read(names[-1]), tensors[names[-1]])


def test_load_model_refuses_without_gpu_or_reports_bad_folder(model_dirs, tmp_path):
    import ninfer_amd
    with pytest.raises(ninfer_amd.ConfigError, match="no such file"):
        ninfer_amd.load_model(str(tmp_path / "empty"))
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="no CPU path"):
            ninfer_amd.load_model(model_dirs["A"]["float32"])


def test_random_weights_are_a_function_of_seed_name_and_index():
    """Every element depends on (seed, tensor name, flat index) alone: a slice of a tensor
    can be computed without the rest, another name or seed gives other numbers, and the
    numbers have the moments of a normal distribution (they are sums of twelve uniform ones)."""
    from ninfer_amd.weights import RandomSource, TensorSpec, counter_random
    specs = {"a.weight": TensorSpec((300, 70)), "b.weight": TensorSpec((300, 70)),
             "n.weight": TensorSpec((64,), "gain")}
    src = RandomSource(specs, 7, torch.float32, std=0.5)
    a = src.read("a.weight")
    assert torch.equal(a, RandomSource({"a.weight": specs["a.weight"]}, 7, torch.float32, std=0.5).read("a.weight"))
    key = counter_random.tensor_key(7, "a.weight")
    part = counter_random.counter_normal(key, 1000, 50)
    assert torch.equal(a.reshape(-1)[1000:1050], torch.from_numpy(part) * 0.5)
    assert not torch.equal(a, src.read("b.weight"))
    assert not torch.equal(a, RandomSource(specs, 8, torch.float32, std=0.5).read("a.weight"))
    z = a / 0.5
    assert abs(float(z.mean())) < 0.02 and abs(float(z.std()) - 1) < 0.02
    assert abs(float((z ** 4).mean()) - 2.9) < 0.15 and float(z.abs().max()) <= 6.0
    gain = src.read("n.weight")
    assert abs(float(gain.mean()) - 1) < 0.3
    bf = RandomSource(specs, 7, torch.bfloat16, std=0.5).read("a.weight")
    assert torch.equal(bf, a.to(torch.bfloat16))
