"""Configuration, registry, weight loading and the random-weights mode (no GPU)."""
import json

import pytest
import torch
from safetensors.torch import save_file

import tiny_models
from torchlet_amd.config import ConfigError, Qwen2Config
from torchlet_amd.models.decoder import DecoderModel
from torchlet_amd.registry import ARCHITECTURES, config_class, load_config
from torchlet_amd.weights.loader import SafetensorsFolder, WeightError, check_against, load_folder
from torchlet_amd.weights.random_init import random_tensors, write_model_folder

# the tiny dictionary configuration of the reference's loader test
# (/root/reference/tests/test_weight_loading.py:75-84): heads of 4
REF_TINY = dict(vocab_size=16, hidden_size=16, num_hidden_layers=1, num_attention_heads=4, num_key_value_heads=2,
                intermediate_size=32, max_position_embeddings=8, tie_word_embeddings=True)


def test_defaults_are_the_references():
    c = Qwen2Config.from_dict(dict(vocab_size=10, hidden_size=32, num_hidden_layers=2, num_attention_heads=4,
                                   intermediate_size=48, max_position_embeddings=64))
    assert (c.num_key_value_heads, c.rms_norm_eps, c.attention_bias, c.rope_theta, c.tie_word_embeddings) == \
           (4, 1e-6, True, 1_000_000.0, False)
    assert c.head_dim == 8 and c.num_kv_groups == 1 and not c.use_sliding_window


def test_rope_parameters_win_over_top_level():
    base = dict(REF_TINY, rope_theta=5.0)
    assert Qwen2Config.from_dict(base).rope_theta == 5.0
    assert Qwen2Config.from_dict(dict(base, rope_parameters={"rope_theta": 7.0})).rope_theta == 7.0


def test_every_size_comes_from_the_keys():
    for name, d in tiny_models.CONFIGS.items():
        c = config_class(d["architectures"][0]).from_dict(d)
        spec = c.to_spec()
        assert spec.vocab_size == d["vocab_size"] and spec.hidden == d["hidden_size"]
        assert len(spec.layers) == d["num_hidden_layers"] == len(spec.order)
        m = spec.layers[0].mixer
        assert (m.num_heads, m.num_kv_heads) == (d["num_attention_heads"], d["num_key_value_heads"])
        assert m.head_dim == d.get("head_dim", d["hidden_size"] // d["num_attention_heads"])
        assert spec.layers[0].ffn.intermediate == d["intermediate_size"]
        assert spec.layers[0].mixer_norm.eps == d.get("rms_norm_eps", 1e-6)          # F leaves it to the default
    c = Qwen2Config.from_dict(tiny_models.CONFIGS["C"])
    assert [l.mixer.window for l in c.to_spec().layers] == [None, 20, 20, 20]
    assert c.rope_theta == 500000.0 and not c.attention_bias


@pytest.mark.parametrize("change,fragment", [
    (dict(hidden_size=None), "hidden_size"),
    (dict(num_key_value_heads=3), "multiple"),
    (dict(head_dim=7), "even"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(rope_scaling={"type": "yarn"}), "rope_scaling"),
    (dict(use_sliding_window=True), "sliding_window"),
    (dict(num_hidden_layers=0), "num_hidden_layers"),
    (dict(rms_norm_eps=0.0), "rms_norm_eps"),
])
def test_bad_configurations_are_refused(change, fragment):
    d = {k: v for k, v in dict(REF_TINY, **change).items() if v is not None}
    with pytest.raises(ConfigError, match=fragment):
        Qwen2Config.from_dict(d)


def test_registry(tmp_path):
    assert "Qwen2ForCausalLM" in ARCHITECTURES
    with pytest.raises(ConfigError, match="not registered.*Qwen2ForCausalLM"):
        config_class("LlamaForCausalLM")
    (tmp_path / "config.json").write_text(json.dumps(dict(REF_TINY, architectures=["Qwen2ForCausalLM"])))
    assert isinstance(load_config(tmp_path), Qwen2Config)
    (tmp_path / "config.json").write_text(json.dumps(REF_TINY))
    with pytest.raises(ConfigError, match="architectures"):
        load_config(tmp_path)


def test_run_order_is_checked():
    from torchlet_amd.config import RunEntry
    spec = Qwen2Config.from_dict(REF_TINY).to_spec()
    import dataclasses
    dataclasses.replace(spec, order=(RunEntry(0), RunEntry(0), RunEntry(0, cache_of=0)))   # a layer twice, a shared cache
    with pytest.raises(ConfigError, match="does not run before"):
        dataclasses.replace(spec, order=(RunEntry(0, cache_of=0),))
    with pytest.raises(ConfigError, match="names layer"):
        dataclasses.replace(spec, order=(RunEntry(1),))


def _model(d, dtype=torch.bfloat16):
    return DecoderModel(Qwen2Config.from_dict(d).to_spec(), dtype, "cpu")


def test_head_sizes_that_no_kernel_takes_are_refused():
    assert _model(REF_TINY).blocks[0].mixer.kernel_libraries() == ["attention_hd16"]        # heads of 4: served by the library of 16
    assert _model(dict(REF_TINY, head_dim=40)).blocks[0].mixer.kernel_libraries() == ["attention_hd48"]
    with pytest.raises(ConfigError, match="even"):
        _model(dict(REF_TINY, head_dim=7))
    with pytest.raises(ConfigError, match="even head sizes from 2 to 256"):
        _model(dict(REF_TINY, head_dim=258))


def test_reference_tiny_config_loads_strictly_in_bf16(tmp_path):
    """Counterpart of the reference's version test (tests/test_weight_loading.py:72-98): bf16
    tensors stay bf16, the tied head *is* the embedding tensor, rotary constants stay 32-bit."""
    cfg = Qwen2Config.from_dict(REF_TINY)
    write_model_folder(cfg, 0, tmp_path)
    src = SafetensorsFolder(tmp_path)
    assert "lm_head.weight" not in src
    assert {src.stored_dtype(n) for n in src} == {"BF16"}
    model = _model(REF_TINY)
    load_folder(model, tmp_path)
    assert model.head is model.embed and model.embed.dtype == torch.bfloat16
    blk = model.blocks[0]
    assert blk.mixer.w_qkv.dtype == torch.bfloat16 and blk.mixer.b_qkv.dtype == torch.bfloat16
    assert blk.mixer_norm.weight.dtype == torch.bfloat16
    assert blk.mixer.position.inv_freq.dtype == torch.float32
    assert blk.mixer.w_qkv.shape == (16 + 2 * 8, 16) and blk.ffn.gate_up.shape == (64, 16)


def test_tensors_stored_in_32_bit_stay_so_and_fp32_engine_widens(tmp_path):
    cfg = Qwen2Config.from_dict(REF_TINY)
    t = random_tensors(cfg, 0, torch.bfloat16)
    t["model.norm.weight"] = t["model.norm.weight"].float()
    t["model.layers.0.self_attn.q_proj.bias"] = t["model.layers.0.self_attn.q_proj.bias"].float()
    save_file(t, str(tmp_path / "model.safetensors"))
    model = _model(REF_TINY)
    load_folder(model, tmp_path)
    assert model.final_norm.weight.dtype == torch.float32            # stored in 32-bit: stays
    assert model.blocks[0].ffn_norm.weight.dtype == torch.bfloat16   # stored in bfloat16: stays
    assert model.blocks[0].mixer.b_qkv.dtype == torch.float32        # mixed parts: widened together
    assert model.blocks[0].mixer.w_qkv.dtype == torch.bfloat16
    m32 = _model(REF_TINY, torch.float32)
    load_folder(m32, tmp_path)
    assert m32.embed.dtype == torch.float32 and m32.blocks[0].ffn_norm.weight.dtype == torch.float32
    torch.testing.assert_close(m32.embed, model.embed.float(), rtol=0, atol=0)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = Qwen2Config.from_dict(REF_TINY)
    t = random_tensors(cfg, 0)
    del t["model.layers.0.mlp.up_proj.weight"], t["model.norm.weight"]
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(2)
    t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(4, 64, dtype=torch.bfloat16)
    save_file(t, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        load_folder(_model(REF_TINY), tmp_path)
    msg = str(e.value)
    assert "missing (2)" in msg and "model.layers.0.mlp.up_proj.weight" in msg and "model.norm.weight" in msg
    assert "unexpected (1)" in msg and "rotary_emb.inv_freq" in msg
    assert "k_proj.weight: stored [4, 64], model wants [8, 16]" in msg
    assert "lm_head.weight" not in msg                       # a tied head may be absent


def test_untied_head_must_be_present_and_copy_of_tied_head_is_accepted(tmp_path):
    untied = dict(REF_TINY, tie_word_embeddings=False)
    t = random_tensors(Qwen2Config.from_dict(REF_TINY), 0)    # has no lm_head
    with pytest.raises(WeightError, match="missing.*lm_head.weight"):
        check_against(_model(untied).weight_specs(), t)
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    check_against(_model(untied).weight_specs(), t)
    check_against(_model(REF_TINY).weight_specs(), t)          # tied model, checkpoint with a copy: fine


def test_no_files_and_duplicate_names(tmp_path):
    with pytest.raises(FileNotFoundError, match="not found safetensors files"):
        SafetensorsFolder(tmp_path)
    save_file({"a": torch.zeros(1)}, str(tmp_path / "x.safetensors"))
    save_file({"a": torch.zeros(1), "b": torch.zeros(1)}, str(tmp_path / "y.safetensors"))
    with pytest.raises(WeightError, match="more than one file.*a "):
        SafetensorsFolder(tmp_path)


def test_random_weights_law_and_reproducibility(tmp_path):
    cfg = Qwen2Config.from_dict(tiny_models.CONFIGS["B"])
    a, b, c = random_tensors(cfg, 1, torch.float32), random_tensors(cfg, 1, torch.float32), random_tensors(cfg, 2, torch.float32)
    assert all(torch.equal(a[k], b[k]) for k in a) and not torch.equal(a["lm_head.weight"], c["lm_head.weight"])
    w = a["model.layers.1.mlp.down_proj.weight"]
    assert abs(float(w.mean())) < 2e-3 and abs(float(w.std()) - 0.02) < 2e-3
    n = a["model.layers.2.input_layernorm.weight"]
    assert abs(float(n.mean()) - 1.0) < 1e-2 and abs(float(n.std()) - 0.02) < 8e-3
    bias = a["model.layers.0.self_attn.k_proj.bias"]
    assert abs(float(bias.std()) - 0.02) < 1e-2
    folder = write_model_folder(cfg, 1, tmp_path / "m")
    assert json.loads((folder / "config.json").read_text())["architectures"] == ["Qwen2ForCausalLM"]
    stored = SafetensorsFolder(folder)
    assert set(stored) == set(a)
    assert torch.equal(stored["lm_head.weight"], a["lm_head.weight"].to(torch.bfloat16))
    assert isinstance(load_config(folder), Qwen2Config)


def test_attention_part_fuses_its_projections_and_keeps_32_bit_biases():
    """q, k and v become one matrix; biases stored in different dtypes are kept in 32-bit; the
    bfloat16 engine reorders the rows of q and k (not v) into the pair layout of the rotary
    encoding, the 32-bit engine leaves them as they are."""
    from torchlet_amd.config import AttentionSpec, RotarySpec
    from torchlet_amd.kernels import ops
    from torchlet_amd.parts import MIXERS
    heads, kvh, hd, hidden = 4, 2, 16, 24
    spec = AttentionSpec(hidden=hidden, num_heads=heads, num_kv_heads=kvh, head_dim=hd, qkv_bias=True,
                         position=RotarySpec(head_dim=hd, theta=1e4, max_positions=64))
    g = torch.Generator().manual_seed(0)
    t = {f"{n}_proj.weight": torch.randn(w * hd, hidden, generator=g).to(torch.bfloat16) for n, w in (("q", heads), ("k", kvh), ("v", kvh))}
    t["o_proj.weight"] = torch.randn(hidden, heads * hd, generator=g).to(torch.bfloat16)
    t["q_proj.bias"] = torch.randn(heads * hd, generator=g)                        # stored in 32-bit
    t["k_proj.bias"] = torch.randn(kvh * hd, generator=g).to(torch.bfloat16)
    t["v_proj.bias"] = torch.randn(kvh * hd, generator=g).to(torch.bfloat16)
    plain_rows = torch.cat([t[f"{n}_proj.weight"] for n in "qkv"])
    plain_bias = torch.cat([t[f"{n}_proj.bias"].float() for n in "qkv"])

    wide = MIXERS.build(spec, torch.float32, torch.device("cpu"))
    wide.load_weights(t)
    assert not wide.pair_layout and torch.equal(wide.w_qkv, plain_rows.float()) and torch.equal(wide.b_qkv, plain_bias)

    half = MIXERS.build(spec, torch.bfloat16, torch.device("cpu"))
    half.load_weights(t)
    assert half.pair_layout and half.b_qkv.dtype == torch.float32 and half.w_qkv.dtype == torch.bfloat16
    order = torch.cat((ops.pair_layout_rows(heads + kvh, hd), (heads + kvh) * hd + torch.arange(kvh * hd)))
    assert torch.equal(half.w_qkv, plain_rows[order]) and torch.equal(half.b_qkv, plain_bias[order])
    # within a head: row 2j is the old row j, row 2j + 1 the old row j + hd/2
    assert order[:6].tolist() == [0, 8, 1, 9, 2, 10] and order[hd:hd + 2].tolist() == [16, 24]


def test_start_up_reports(tmp_path):
    """The reports the reference logs when an LLM starts (llm.py:28-36): one line per tensor with name, shape and
    stored type, and a description of the backend; a logger that stands at WARNING unless asked."""
    import io
    import logging

    from torchlet_amd.logger import backend_info, get_logger, weights_info
    cfg = Qwen2Config.from_dict(REF_TINY)
    write_model_folder(cfg, 0, tmp_path)
    lines = weights_info(SafetensorsFolder(tmp_path)).splitlines()
    assert len(lines) == len(random_tensors(cfg, 0)) and any(l.split() == ["model.norm.weight", "[16]", "BF16"] for l in lines)
    assert weights_info({"a": torch.zeros(2, 3)}) == "a  [2, 3]  torch.float32"
    assert "torch:" in backend_info() and "gfx950" in backend_info()
    stream = io.StringIO()
    log = get_logger("torchlet_amd.test", stream=stream)
    log.info("hidden")
    assert stream.getvalue() == "" and log.level == logging.WARNING
    get_logger("torchlet_amd.test", level=logging.INFO).info("shown %d", 3)
    assert "[INFO] torchlet_amd.test" in stream.getvalue() and "shown 3" in stream.getvalue()


def test_compute_dtype_follows_the_folder(tmp_path):
    """The reference types its parameters and its cache after the checkpoint's tensors
    (/root/reference/src/torchlet/utils.py:18-38, v10_triton_paged_gqa/engine.py:58): a folder stored in
    32-bit runs in 32-bit.  Here the folder's ``torch_dtype`` decides, else what it stores; a named
    dtype converts at load; anything but bfloat16 and float32 is refused by name."""
    from torchlet_amd.engine.loading import load_model, resolve_dtype
    cfg = Qwen2Config.from_dict(REF_TINY)
    assert cfg.torch_dtype == "" and cfg.to_dict()["torch_dtype"] is None
    f32 = write_model_folder(cfg, 0, tmp_path / "f32", torch.float32)
    bf16 = write_model_folder(cfg, 0, tmp_path / "bf16", torch.bfloat16)
    assert json.loads((f32 / "config.json").read_text())["torch_dtype"] == "float32"
    assert resolve_dtype(f32, load_config(f32)) == "float32" and resolve_dtype(bf16, load_config(bf16)) == "bfloat16"
    for folder in (f32, bf16):                       # without the key: the stored element type decides
        d = json.loads((folder / "config.json").read_text())
        del d["torch_dtype"]
        (folder / "config.json").write_text(json.dumps(d))
    assert resolve_dtype(f32, load_config(f32)) == "float32" and resolve_dtype(bf16, load_config(bf16)) == "bfloat16"
    assert resolve_dtype(f32, load_config(f32), "bfloat16") == "bfloat16"       # named: converts at load
    assert resolve_dtype(bf16, load_config(bf16), torch.float32) == "float32"
    _, model = load_model(f32, device="cpu")
    assert model.dtype == torch.float32 and model.embed.dtype == torch.float32 and model.blocks[0].mixer.w_qkv.dtype == torch.float32
    _, model = load_model(bf16, device="cpu")
    assert model.dtype == torch.bfloat16 and model.embed.dtype == torch.bfloat16
    _, model = load_model(f32, "bfloat16", device="cpu")
    assert model.dtype == torch.bfloat16 and model.blocks[0].ffn.down.dtype == torch.bfloat16
    # a dtype for which no engine is built: refused by its name, from the key and from the stored tensors
    d = json.loads((bf16 / "config.json").read_text())
    (bf16 / "config.json").write_text(json.dumps(dict(d, torch_dtype="float16")))
    with pytest.raises(ValueError, match="float16"):
        load_model(bf16, device="cpu")
    f16 = write_model_folder(cfg, 0, tmp_path / "f16", torch.float16)
    d = json.loads((f16 / "config.json").read_text())
    del d["torch_dtype"]
    (f16 / "config.json").write_text(json.dumps(d))
    with pytest.raises(ValueError, match="float16"):
        load_model(f16, device="cpu")
    assert load_model(f16, "float32", device="cpu")[1].dtype == torch.float32


def test_dtype_policy_of_a_tensor_is_apart_from_its_shape_and_laws_are_named():
    from torchlet_amd.parts.base import INIT_LAWS, WeightSpec, place, register_init_law
    m = torch.randn(3, 5).to(torch.bfloat16)
    assert place(m, "compute", torch.bfloat16, "cpu").dtype == torch.bfloat16
    assert place(m, "float32", torch.bfloat16, "cpu").dtype == torch.float32            # a matrix that stays 32-bit
    assert place(m.float(), "stored", torch.bfloat16, "cpu").dtype == torch.float32     # stored in 32-bit: stays
    assert place(m, "stored", torch.float32, "cpu").dtype == torch.float32              # a 32-bit engine widens
    assert place(m.half(), "stored", torch.bfloat16, "cpu").dtype == torch.float32      # neither of the two: widened
    assert place(torch.arange(4), "int32", torch.bfloat16, "cpu").dtype == torch.int32
    for bad in (dict(keep="vector"), dict(init="no_such_law")):
        with pytest.raises(ConfigError):
            WeightSpec((2, 2), **bad)
    with pytest.raises(ConfigError):
        place(m, "matrix", torch.bfloat16, "cpu")
    register_init_law("test_all_sevens")(lambda shape, gen, device, std: torch.full(shape, 7.0, device=device))
    try:
        assert WeightSpec((2,), init="test_all_sevens").init == "test_all_sevens"
        assert float(INIT_LAWS["test_all_sevens"]((2,), None, "cpu", 0.02).sum()) == 14.0
    finally:
        INIT_LAWS.pop("test_all_sevens")


def test_every_part_is_asked_whether_a_step_may_be_recorded():
    """Not the mixers alone: a feed-forward, a norm or a position encoding that reads values of the step on the host
    keeps the whole model off graphs.  ``False`` is the default of a part; the built-in parts say ``True``."""
    from torchlet_amd.parts import FeedForward, Part
    from torchlet_amd.parts.base import LazyNorm, Stream
    assert Part.graph_safe is False
    model = _model(REF_TINY)
    kinds = {type(p).__name__ for p in model.parts()}
    assert kinds == {"PreNormBlock", "RMSNorm", "GQAttention", "RotaryEncoding", "SwiGLU"} and model.graph_safe()

    class HostReadingFFN(FeedForward):
        def forward(self, h, ctx):
            return h
    model.blocks[0].ffn = model.blocks[0]._children["mlp"] = HostReadingFFN(None, torch.bfloat16, "cpu")
    assert not model.graph_safe()
    # a norm that has not run yet names its kind, and only a root-mean-square norm hands out (weight, eps)
    norm = model.final_norm
    norm.weight = torch.ones(16)
    lazy = LazyNorm(norm, Stream(torch.zeros(1, 16)), "rmsnorm", weight=norm.weight, eps=norm.eps)
    assert lazy.rmsnorm() == (norm.weight, norm.eps)
    assert LazyNorm(norm, Stream(torch.zeros(1, 16)), "layernorm", weight=norm.weight, bias=None, eps=1e-5).rmsnorm() is None
