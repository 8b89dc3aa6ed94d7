"""Configuration, registry, safetensors reading and writing, weight errors (no GPU)."""
from __future__ import annotations

import json
import os

import pytest
import torch

from serve_amd.config.llama import ConfigError, LlamaConfig
from serve_amd.models.model import Model
from serve_amd.parts.base import Runtime
from serve_amd.registry import get_architecture, known_architectures, load_config
from serve_amd.weights import loader
from serve_amd.weights.safetensors_io import CheckpointReader, DictReader, write_safetensors
from tests import util


def hf(**over):
    d = util.TINY_B.to_hf_dict()
    d.update(over)
    return d


def test_config_round_trip_and_defaults():
    for cfg in (util.TINY_A, util.TINY_B, util.TINY_C):
        assert LlamaConfig.from_hf_dict(cfg.to_hf_dict()) == cfg
    d = hf()
    for k in ("num_key_value_heads", "head_dim", "rms_norm_eps", "rope_theta", "rope_scaling", "tie_word_embeddings"):
        d.pop(k)
    c = LlamaConfig.from_hf_dict(d)
    # defaults of the reference's ModelArgs: serve/model.py:29-30; head_dim = dim // n_heads (:91)
    assert (c.num_key_value_heads, c.head_dim, c.rms_norm_eps, c.rope_theta) == (3, 32, 1e-5, 10000.0)
    assert c.rope_scaling is None and c.tie_word_embeddings is False


def test_head_dim_need_not_be_hidden_over_heads():
    c = LlamaConfig.from_hf_dict(hf(head_dim=48))
    spec = get_architecture("LlamaForCausalLM").build_spec(c)
    shapes = {r.checkpoint_name: r.shape for r in Model(spec).weight_requests()}
    assert shapes["model.layers.0.self_attn.q_proj.weight"] == (3 * 48, 96)
    assert shapes["model.layers.0.self_attn.o_proj.weight"] == (96, 3 * 48)


@pytest.mark.parametrize("over,word", [
    (dict(attention_bias=True), "bias"), (dict(mlp_bias=True), "bias"), (dict(hidden_act="gelu"), "hidden_act"),
    (dict(rope_scaling=dict(rope_type="yarn", factor=2.0)), "rope_type"),
    (dict(rope_scaling=dict(rope_type="llama3", factor=2.0)), "lacks"),
    (dict(num_key_value_heads=2), "multiple"), (dict(head_dim=33), "even"), (dict(vocab_size=0), "positive"),
])
def test_config_refuses(over, word):
    with pytest.raises(ConfigError, match=word):
        LlamaConfig.from_hf_dict(hf(**over))


def test_config_missing_keys_are_named():
    d = hf()
    d.pop("intermediate_size")
    d.pop("vocab_size")
    with pytest.raises(ConfigError, match="intermediate_size") as e:
        LlamaConfig.from_hf_dict(d)
    assert "vocab_size" in str(e.value)


def test_registry(tmp_path):
    assert "LlamaForCausalLM" in known_architectures()
    with pytest.raises(KeyError, match="LlamaForCausalLM"):
        get_architecture("NopeForCausalLM")
    folder = util.make_folder(tmp_path, "B")
    arch, cfg = load_config(folder)
    assert arch.name == "LlamaForCausalLM" and cfg == util.TINY_B
    with pytest.raises(FileNotFoundError):
        load_config(str(tmp_path / "nothing"))


def test_spec_is_data():
    spec = get_architecture("LlamaForCausalLM").build_spec(util.TINY_A)
    assert [e.layer for e in spec.run_order] == [0, 1] and [e.cache for e in spec.run_order] == [0, 1]
    assert spec.layers[0].parts["mixer"].kind == "gqa_attention" and spec.layers[1].parts["ffn"].kind == "swiglu"
    assert spec.layers[1].parts["mixer"].params["position"].params["theta"] == 10000.0
    m = Model(spec)
    assert len(m.cache_requests()) == 2 and m.state_requests() == [None, None]


def test_safetensors_round_trip_with_the_library(tmp_path):
    from safetensors.torch import load_file, save_file
    t = {"a": torch.randn(3, 5).bfloat16(), "b": torch.arange(7, dtype=torch.int64), "c": torch.randn(2, 2, 2),
         "s": torch.tensor(3.5)}
    p = str(tmp_path / "x.safetensors")
    write_safetensors(p, t.items())
    back = load_file(p)                       # the library reads what we write
    for k in t:
        assert back[k].dtype == t[k].dtype and torch.equal(back[k], t[k])
    p2 = str(tmp_path / "model.safetensors")
    save_file(t, p2)                          # and we read what the library writes
    r = CheckpointReader(str(tmp_path))
    assert sorted(r.names()) == sorted(t)
    for k in t:
        dt, shape = r.info(k)
        assert dt == t[k].dtype and shape == tuple(t[k].shape) and torch.equal(r.read(k), t[k])


def test_sharded_folder(tmp_path):
    a, b = {"x": torch.ones(2)}, {"y": torch.zeros(3)}
    write_safetensors(str(tmp_path / "m-1.safetensors"), a.items())
    write_safetensors(str(tmp_path / "m-2.safetensors"), b.items())
    with open(tmp_path / "model.safetensors.index.json", "w") as f:
        json.dump({"weight_map": {"x": "m-1.safetensors", "y": "m-2.safetensors"}}, f)
    r = CheckpointReader(str(tmp_path))
    assert sorted(r.names()) == ["x", "y"] and torch.equal(r.read("y"), torch.zeros(3))
    with pytest.raises(FileNotFoundError):
        CheckpointReader(str(tmp_path / "none"))


def test_random_folder_is_a_function_of_seed_and_name(tmp_path):
    f1 = loader.write_random_model(str(tmp_path / "a"), util.TINY_B, 1)
    f2 = loader.write_random_model(str(tmp_path / "b"), util.TINY_B, 1)
    f3 = loader.write_random_model(str(tmp_path / "c"), util.TINY_B, 2)
    w1, w2, w3 = util.plain_weights(f1), util.plain_weights(f2), util.plain_weights(f3)
    assert sorted(w1) == sorted(w2) and all(torch.equal(w1[k], w2[k]) for k in w1)
    assert not torch.equal(w1["model.norm.weight"], w3["model.norm.weight"])
    assert "lm_head.weight" not in w1                       # tied: no output matrix is written
    assert "lm_head.weight" in util.plain_weights(util.make_folder(tmp_path, "A"))
    assert all(v.dtype == torch.bfloat16 for v in w1.values())
    n = w1["model.norm.weight"].float()
    e = w1["model.embed_tokens.weight"].float()
    assert abs(n.mean().item() - 1) < 0.05 and abs(e.std().item() - 0.02) < 0.002
    assert util.plain_config(f1)["architectures"] == ["LlamaForCausalLM"]


def model_of(cfg):
    return Model(get_architecture("LlamaForCausalLM").build_spec(cfg))


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    m = model_of(util.TINY_A)
    t = dict(loader.random_tensors(m, 0))
    t.pop("model.layers.1.mlp.up_proj.weight")
    t.pop("model.norm.weight")
    t["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 63, dtype=torch.bfloat16)
    t["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(16)
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)      # known and ignored
    with pytest.raises(loader.WeightError) as e:
        loader.check_against(m, DictReader(t))
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.q_norm.weight"]
    assert err.wrong_shape == [("model.layers.0.self_attn.q_proj.weight", (64, 63), (64, 64))]
    text = str(err)
    for word in ("missing", "unexpected", "wrong shape", "up_proj", "q_norm", "[64, 63]", "[64, 64]"):
        assert word in text


def test_untied_model_without_output_matrix_is_missing_nothing_but_shares_the_table():
    # a checkpoint without lm_head.weight shares the embedding table, tied flag or not
    m = model_of(util.TINY_A)
    t = dict(loader.random_tensors(m, 0))
    t.pop("lm_head.weight")
    loader.check_against(m, DictReader(t))
    # a tied model may still carry the matrix
    mb = model_of(util.TINY_B)
    tb = dict(loader.random_tensors(mb, 0))
    tb["lm_head.weight"] = tb["model.embed_tokens.weight"].clone()
    loader.check_against(mb, DictReader(tb))


def test_dtype_rule():
    bf, f32 = Runtime.__new__(Runtime), Runtime.__new__(Runtime)
    bf.dtype, f32.dtype = torch.bfloat16, torch.float32
    assert loader.device_dtype(torch.bfloat16, bf) == torch.bfloat16
    assert loader.device_dtype(torch.float16, bf) == torch.bfloat16
    assert loader.device_dtype(torch.float32, bf) == torch.float32       # stored in 32-bit stays so
    assert loader.device_dtype(torch.bfloat16, f32) == torch.float32
    assert loader.device_dtype(torch.int64, bf) == torch.int32 and loader.device_dtype(torch.int16, f32) == torch.int32


def test_engine_refuses_to_run_without_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("a GPU is here")
    from serve_amd.engine.engine import Engine
    with pytest.raises(RuntimeError, match="GPU"):
        Engine.from_config(util.TINY_A, 0)


def test_bench_refuses_more_than_one_gpu():
    """The engine runs on one GPU: for another count bench.py prints one line that says so and
    exits with 2 (before it touches torch or the GPU)."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True,
                          text=True, timeout=60)
    assert proc.returncode == 2
    assert len(proc.stdout.strip().splitlines()) == 1 and "one GPU" in proc.stdout


def test_config_json_of_a_checkpoint_with_all_its_keys():
    """config.json as checkpoints ship it: keys the engine has no use for are ignored, absent
    head_dim and num_key_value_heads take their defaults, "default" rope scaling means none."""
    hf = {"architectures": ["LlamaForCausalLM"], "attention_bias": False, "attention_dropout": 0.0,
          "bos_token_id": 128000, "eos_token_id": [128001, 128008], "hidden_act": "silu", "hidden_size": 96,
          "initializer_range": 0.02, "intermediate_size": 200, "max_position_embeddings": 4096, "mlp_bias": False,
          "model_type": "llama", "num_attention_heads": 6, "num_hidden_layers": 2, "pretraining_tp": 1,
          "rms_norm_eps": 1e-05, "rope_scaling": {"rope_type": "default"}, "rope_theta": 500000.0,
          "torch_dtype": "bfloat16", "transformers_version": "4.45.0", "use_cache": True, "vocab_size": 300}
    cfg = LlamaConfig.from_hf_dict(hf)
    assert (cfg.head_dim, cfg.num_key_value_heads, cfg.rope_scaling, cfg.tie_word_embeddings) == (16, 6, None, False)
    hf["rope_scaling"] = {"type": "linear", "factor": 2.0}
    with pytest.raises(Exception, match="linear"):
        LlamaConfig.from_hf_dict(hf)


def test_attention_key_splits_are_chosen_by_the_shape_of_the_launch():
    """Whole prompts are never cut (the causal mask makes the parts unequal), short portions of long
    contexts and steps of decoded tokens are, until the chip is filled."""
    from serve_amd.ops import attention_splits
    assert attention_splits(2048, 1, 8, 2048, 4) == 1
    assert attention_splits(1024, 2, 8, 1500, 4) == 1
    assert attention_splits(512, 1, 8, 4096, 4) == 2
    assert attention_splits(128, 1, 8, 4096, 4) == 4
    assert attention_splits(256, 1, 8, 1024, 4) == 1           # parts would be shorter than 1024 keys
    assert attention_splits(512, 8, 8, 4096, 4) == 1           # enough workgroups already
    assert attention_splits(1, 8, 8, 4096) == 8
    assert attention_splits(1, 64, 8, 300) == 1
    assert attention_splits(1, 1, 8, 100000) == 64


def test_named_shapes_are_the_configurations_the_measurements_are_specified_on():
    """`--shape tiny-a | tiny-b | llama-1b | llama-3b | llama-8b`: the presets hold the sizes that the
    measured configurations are specified with (two tiny ones that differ in every size and option,
    and the shapes of Llama-3.2-1B, Llama-3.2-3B and Llama-3.1-8B)."""
    from serve_amd.benchmark import SHAPES
    a, b, one = SHAPES["tiny-a"], SHAPES["tiny-b"], SHAPES["llama-1b"]
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim,
            a.intermediate_size, a.vocab_size, a.rope_theta, a.rope_scaling, a.rms_norm_eps, a.tie_word_embeddings) == \
        (2, 64, 4, 2, 16, 192, 256, 10000.0, None, 1e-5, False)
    assert (b.num_hidden_layers, b.hidden_size, b.num_attention_heads, b.num_key_value_heads, b.head_dim,
            b.intermediate_size, b.vocab_size, b.rope_theta, b.rms_norm_eps, b.tie_word_embeddings) == \
        (3, 96, 3, 1, 32, 256, 512, 500000.0, 1e-6, True)
    s = b.rope_scaling
    assert (s.factor, s.low_freq_factor, s.high_freq_factor, s.original_max_position_embeddings) == (32.0, 1.0, 4.0, 64)
    assert (one.num_hidden_layers, one.hidden_size, one.num_attention_heads, one.num_key_value_heads, one.head_dim,
            one.intermediate_size, one.vocab_size, one.tie_word_embeddings) == (16, 2048, 32, 8, 64, 8192, 128256, True)
    assert SHAPES["llama-3b"].num_hidden_layers == 28 and SHAPES["llama-8b"].intermediate_size == 14336
    for cfg in SHAPES.values():
        cfg.validate()


def test_attention_launch_policy_is_the_same_for_a_step_and_its_graph_replay():
    """A decode step replayed from a graph sees its batch padded to the next captured size and its
    longest context rounded up to a power of two; the choice of key splits and of the cut inside a
    workgroup must not change with that, or a replay would differ from the eager step."""
    import random
    from serve_amd import ops
    from serve_amd.engine.runner import GRAPH_BATCHES
    rng = random.Random(5)
    for _ in range(2000):
        B = rng.randrange(1, GRAPH_BATCHES[-1] + 1)
        ctx = rng.randrange(1, 140000)
        Hk, G = rng.choice([1, 2, 4, 8]), rng.choice([1, 3, 4, 8])
        b_pad = next(b for b in GRAPH_BATCHES if b >= B)
        bucket = 256
        while bucket < ctx:
            bucket *= 2
        assert ops.attention_splits(1, B, Hk, ctx, G) == ops.attention_splits(1, b_pad, Hk, bucket, G)
        assert ops.attention_in_workgroup(1, B, ctx, G) == ops.attention_in_workgroup(1, b_pad, bucket, G)


def test_rotary_part_refuses_contexts_beyond_its_kernels_angles():
    """The bfloat16 kernels reduce the rotation angle themselves and hold up to 4e6 rad: a
    longer context is refused when the part is loaded, not rotated wrongly (float32 has no limit)."""
    import pytest
    from serve_amd.parts.base import Runtime
    from serve_amd.parts.standard import RotaryPosition
    part = RotaryPosition(head_dim=64, rot_dim=64, theta=500000.0)
    with pytest.raises(ValueError, match="rotation angles"):
        part.load({}, Runtime(torch.device("cpu"), torch.bfloat16, max_context=8_000_000))
    part.load({}, Runtime(torch.device("cpu"), torch.bfloat16, max_context=1_000_000))
    part.load({}, Runtime(torch.device("cpu"), torch.float32, max_context=8_000_000))
    assert part.rotary().rot_dim == 64 and not part.rotary().adjacent_pairs


def test_command_line_writes_a_random_model_and_knows_the_short_names(tmp_path):
    """`random-model` needs no GPU: a folder from a named shape (`--preset` is another name of
    `--shape`), readable by the loader's own reader; `bf16` and `fp32` are other names of the dtypes."""
    from serve_amd.__main__ import dtype_name, main
    from serve_amd.registry import load_config
    from serve_amd.weights.safetensors_io import CheckpointReader
    assert dtype_name("bf16") == "bfloat16" and dtype_name("fp32") == "float32" and dtype_name("float32") == "float32"
    out = str(tmp_path / "m")
    assert main(["random-model", "--preset", "tiny-a", "--out", out, "--seed", "4", "--weight-dtype", "float32"]) == 0
    _, cfg = load_config(out)
    assert cfg.hidden_size == 64 and cfg.num_hidden_layers == 2
    reader = CheckpointReader(out)
    assert "model.embed_tokens.weight" in reader.names()
    assert main(["no-such-command"]) == 2


def test_measurement_prices_a_step_by_the_parts_own_accounts():
    """`bench.py` takes the bytes a decode step reads and the flops of a prompt from the model
    (`Model.step_cost`, `Model.cache_elements_per_token`, which add up what each part says of itself).
    For the dense decoder they are the sums one writes down by hand: per layer the four attention
    matrices, the three of the feed-forward and two norm vectors; the output matrix once (tied or not:
    the embedding's rows are gathered, not streamed) and the last norm; keys and values of every layer
    per cached token; for a prompt of T tokens two flops per matrix element and token, the output matrix
    for one row, and four flops per head dim, query head and visible key."""
    import bench
    from serve_amd.benchmark import SHAPES
    for name in ("llama-1b", "llama-3b", "llama-8b", "tiny-a", "tiny-b"):
        cfg = SHAPES[name]
        model = Model(get_architecture(cfg.architecture).build_spec(cfg))
        d, D, L = cfg.hidden_size, cfg.head_dim, cfg.num_hidden_layers
        matrices = ((cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * D * d + d * cfg.num_attention_heads * D
                    + 3 * d * cfg.intermediate_size)
        assert bench.weight_bytes(model, 2) == 2 * ((matrices + 2 * d) * L + cfg.vocab_size * d + d)
        assert bench.kv_bytes(model, 384, 2) == 384 * 2 * L * cfg.num_key_value_heads * D * 2
        T = 2048
        want = 2.0 * matrices * L * T + 2.0 * cfg.vocab_size * d + 4.0 * cfg.num_attention_heads * D * L * (T * (T + 1) / 2)
        assert bench.prefill_flops(model, T) == want
    assert bench.weight_bytes(Model(get_architecture("LlamaForCausalLM").build_spec(SHAPES["llama-1b"])), 2) == 2471628800
    # a portion over earlier keys, and a window: the attention's own account
    from serve_amd.parts.standard import GQAAttention
    from serve_amd.config.spec import PartSpec
    pos = PartSpec("rope", {"head_dim": 16, "rot_dim": 16, "theta": 10000.0})
    proj = 2.0 * 5 * (64 * 64 + 2 * 32 * 64 + 64 * 64)
    full = GQAAttention(64, 4, 2, 16, 0.25, pos).step_cost(5, context_before=10)
    assert full.flops == proj + 4.0 * 4 * 16 * (11 + 12 + 13 + 14 + 15)
    windowed = GQAAttention(64, 4, 2, 16, 0.25, pos, window=12).step_cost(5, context_before=10)
    assert windowed.flops == proj + 4.0 * 4 * 16 * (11 + 12 + 12 + 12 + 12)


def test_float32_products_of_a_few_dozen_rows_leave_no_part_of_k_without_stages():
    """The float32 product for 9 to 128 rows cuts its inner dimension into parts across workgroups, in
    stages of 256 columns spread evenly: with no more parts than stages no part is empty (an empty part
    stores zeros and reads the matrix's last stage, in range; this only says that none is chosen)."""
    from serve_amd import ops
    for K in (512, 1024, 2048, 2304, 3072, 4096, 5120, 8192, 14336):
        for N in (512, 1024, 2048, 2304, 3072, 4096):
            for M in (9, 16, 64, 65, 128):
                parts = ops.f32_mid_parts(M, N, K)
                stages = -(-K // 256)
                assert 1 <= parts <= 8 and parts <= stages
                assert all((z + 1) * stages // parts - z * stages // parts >= 1 for z in range(parts))
