"""Configuration, registry and weight-loading errors (no GPU)."""
import json

import pytest
import torch

from jax_vllm_amd.config import ConfigError, EngineConfig, resolve, supported_architectures
from jax_vllm_amd.models.qwen3 import Qwen3Config
from jax_vllm_amd.parts import DecoderModel, LayerRun, ModelSpec
from jax_vllm_amd.weights.loader import WeightsError, check_against_specs
from jax_vllm_amd.weights.random_init import write_random_model
from jax_vllm_amd.weights.safetensors_io import SafetensorsFile, write_safetensors
from tests.tiny import ALL_TINY, TINY_A, TINY_B, tensor_shapes


def test_config_reads_reference_keys_and_defaults():
    """Keys and defaults of jllm/model/qwen3.py:43-55."""
    c = dict(TINY_B["config"])
    cfg = Qwen3Config.from_dict(c)
    assert (cfg.num_heads, cfg.num_kv_heads, cfg.head_dim) == (6, 2, 32)
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-5 and cfg.tie_word_embeddings is False
    for k in ("num_key_value_heads", "head_dim", "rope_theta", "tie_word_embeddings"):
        del c[k]
    d = Qwen3Config.from_dict(c)
    assert d.num_kv_heads == 6 and d.head_dim == 96 // 6 and d.rope_theta == 1_000_000.0
    assert d.tie_word_embeddings is False


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "rms_norm_eps", "max_position_embeddings"])
def test_config_missing_required_key(key):
    c = dict(TINY_A["config"])
    del c[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(c)


def test_config_validation():
    bad = dict(TINY_A["config"], num_key_value_heads=3)
    with pytest.raises(ConfigError, match="multiple"):
        Qwen3Config.from_dict(bad)
    with pytest.raises(ConfigError, match="even"):
        Qwen3Config.from_dict(dict(TINY_A["config"], head_dim=15))
    with pytest.raises(ConfigError, match="positive"):
        Qwen3Config.from_dict(dict(TINY_A["config"], vocab_size=0))
    with pytest.raises(ConfigError, match="must be int"):
        Qwen3Config.from_dict(dict(TINY_A["config"], hidden_size="64"))
    for key, val in (("use_sliding_window", True), ("rope_scaling", {"type": "yarn"}), ("attention_bias", True),
                     ("hidden_act", "gelu")):
        with pytest.raises(ConfigError, match=key):
            Qwen3Config.from_dict(dict(TINY_A["config"], **{key: val}))


def test_registry_errors_match_reference_wording():
    """jllm/model/weights.py:59-65 and :161-170."""
    assert supported_architectures() == ["Qwen3ForCausalLM"]
    with pytest.raises(ConfigError, match="no 'architectures' field"):
        resolve({k: v for k, v in TINY_A["config"].items() if k != "architectures"})
    with pytest.raises(ConfigError, match="unsupported architecture: 'Qwen2ForCausalLM'.*Supported: Qwen3ForCausalLM"):
        resolve(dict(TINY_A["config"], architectures=["Qwen2ForCausalLM"]))


@pytest.mark.parametrize("tiny", ALL_TINY, ids=[t["name"] for t in ALL_TINY])
def test_model_declares_the_checkpoint_tensors(tiny):
    """Names and shapes of jllm/model/weights.py:118-152; a tied head declares no tensor."""
    arch, cfg, _ = resolve(tiny["config"])
    model = DecoderModel(arch.build_spec(cfg))
    got = {k: tuple(v.shape) for k, v in model.tensor_specs().items()}
    assert got == tensor_shapes(tiny["config"])
    assert ("lm_head.weight" in model.ignored_tensor_names()) == tiny["config"]["tie_word_embeddings"]
    roles = {k: v.role for k, v in model.tensor_specs().items()}
    assert all((r == "vector") == k.endswith("norm.weight") or "layernorm" in k for k, r in roles.items())


def test_engine_config_names_and_checks():
    """Reference names keep their meaning (jllm/engine/engine.py:63-94)."""
    e = EngineConfig(dtype="bf16", block_size=16, max_num_seqs=4, max_model_len=2048)
    assert e.dtype == "bfloat16" and e.usable_pages == 4 * 128 and e.prompt_limit == 2048
    assert EngineConfig(dtype="fp32").dtype == "float32"
    assert EngineConfig(num_blocks=9).usable_pages == 8          # num_blocks counts the null page
    with pytest.raises(ConfigError, match="dtype"):
        EngineConfig(dtype="fp16")
    with pytest.raises(ConfigError, match="max_prefill_len"):
        EngineConfig(max_model_len=64, max_prefill_len=128)
    with pytest.raises(ConfigError, match="num_blocks"):
        EngineConfig(num_blocks=1)


def test_random_model_folder_is_reproducible_and_distributed_as_said(tmp_path):
    a = write_random_model(tmp_path / "a", TINY_B["config"], seed=5, std=0.05, norm_std=0.1)
    b = write_random_model(tmp_path / "b", TINY_B["config"], seed=5, std=0.05, norm_std=0.1)
    c = write_random_model(tmp_path / "c", TINY_B["config"], seed=6, std=0.05, norm_std=0.1)
    fa, fb, fc = (SafetensorsFile(p / "model.safetensors") for p in (a, b, c))
    assert json.loads((a / "config.json").read_text())["architectures"] == ["Qwen3ForCausalLM"]
    assert {k: v[1] for k, v in fa.entries.items()} == tensor_shapes(TINY_B["config"])
    for name in fa.entries:
        assert fa.entries[name][0] == torch.bfloat16
        assert torch.equal(fa.tensor(name), fb.tensor(name))
    w = fa.tensor("model.layers.1.mlp.up_proj.weight").float()
    assert abs(w.mean().item()) < 0.005 and abs(w.std().item() - 0.05) < 0.005
    n = fa.tensor("model.layers.1.self_attn.q_norm.weight").float()
    assert abs(n.mean().item() - 1.0) < 0.08 and 0.03 < n.std().item() < 0.2
    assert not torch.equal(fa.tensor("model.norm.weight"), fc.tensor("model.norm.weight"))
    # any subset is reproducible: a tensor does not depend on which others are generated
    fewer = dict(TINY_B["config"], num_hidden_layers=1)
    d = write_random_model(tmp_path / "d", fewer, seed=5, std=0.05, norm_std=0.1)
    fd = SafetensorsFile(d / "model.safetensors")
    assert torch.equal(fd.tensor("model.layers.0.mlp.down_proj.weight"), fa.tensor("model.layers.0.mlp.down_proj.weight"))


def test_safetensors_round_trip_and_library_compatibility(tmp_path):
    from safetensors.torch import load_file, save_file

    t = {"a": torch.arange(12, dtype=torch.float32).reshape(3, 4), "b": torch.randn(5).to(torch.bfloat16),
         "c": torch.arange(6, dtype=torch.int32)}
    write_safetensors(tmp_path / "mine.safetensors", [(k, tuple(v.shape), v.dtype, lambda v=v: v) for k, v in t.items()])
    theirs = load_file(str(tmp_path / "mine.safetensors"))       # the library reads what we write
    save_file(t, str(tmp_path / "theirs.safetensors"))
    f = SafetensorsFile(tmp_path / "theirs.safetensors")          # and we read what it writes
    for k, v in t.items():
        assert torch.equal(theirs[k], v) and torch.equal(f.tensor(k), v)


def test_weight_errors_list_everything_at_once():
    arch, cfg, _ = resolve(TINY_A["config"])
    model = DecoderModel(arch.build_spec(cfg))
    specs = model.tensor_specs()
    available = {k: (torch.bfloat16, tuple(v.shape)) for k, v in specs.items()}
    check_against_specs("x", specs, model.ignored_tensor_names(), dict(available, **{"lm_head.weight": (torch.bfloat16, (256, 64))}))
    del available["model.layers.1.self_attn.k_norm.weight"]
    del available["model.norm.weight"]
    available["model.layers.0.mlp.up_proj.weight"] = (torch.bfloat16, (64, 128))
    available["model.layers.7.mlp.up_proj.weight"] = (torch.bfloat16, (128, 64))
    available["model.embed_tokens.weight"] = (torch.int64, (256, 64))
    with pytest.raises(WeightsError) as e:
        check_against_specs("ckpt", specs, set(), available)
    msg = str(e.value)
    assert "missing tensors (2): model.layers.1.self_attn.k_norm.weight, model.norm.weight" in msg
    assert "unexpected tensors (1): model.layers.7.mlp.up_proj.weight" in msg
    assert "wrong shape: model.layers.0.mlp.up_proj.weight is [64, 128], the model needs [128, 64]" in msg
    assert "wrong type: model.embed_tokens.weight is stored as int64" in msg
    assert e.value.missing == ["model.layers.1.self_attn.k_norm.weight", "model.norm.weight"]


def test_unused_tensors_are_named_and_tolerated_unless_strict(tmp_path, capsys):
    """jllm/model/weights.py:21-37 reads every tensor of the folder into a dictionary and the
    model asks it only for the names it uses: leftovers (a stored inv_freq buffer, an extra
    head) do not stop a load.  Here they are named on standard error; ``strict`` refuses them;
    a missing tensor stays an error and the error lists the unused ones too."""
    from jax_vllm_amd.weights.loader import load_model

    folder = write_random_model(tmp_path / "m", TINY_A["config"], seed=0, std=0.02, norm_std=0.02)
    f = SafetensorsFile(folder / "model.safetensors")
    items = [(n, tuple(shape), dtype, (lambda n=n: f.tensor(n))) for n, (dtype, shape) in f.entries.items()]
    extra = "model.layers.0.self_attn.rotary_emb.inv_freq"
    items.append((extra, (8,), torch.float32, lambda: torch.arange(8, dtype=torch.float32)))
    write_safetensors(folder / "model.safetensors.new", items)
    f.close()
    (folder / "model.safetensors.new").rename(folder / "model.safetensors")
    model, cfg = load_model(folder, "float32", "cpu")
    err = capsys.readouterr().err
    assert "1 tensor(s) not used by the model: " + extra in err
    assert model.layers[0].mixer.w_qkv.shape == (4 * 16 + 2 * 2 * 16, 64)
    with pytest.raises(WeightsError, match="unexpected tensors \\(1\\): " + extra):
        load_model(folder, "float32", "cpu", strict=True)
    # without strict the checker hands the names back and raises only for real problems
    arch, c, _ = resolve(TINY_A["config"])
    specs = DecoderModel(arch.build_spec(c)).tensor_specs()
    available = {k: (torch.bfloat16, tuple(v.shape)) for k, v in specs.items()}
    available[extra] = (torch.float32, (8,))
    assert check_against_specs("x", specs, set(), available) == [extra]
    del available["model.norm.weight"]
    with pytest.raises(WeightsError) as e:
        check_against_specs("x", specs, set(), available)
    assert e.value.missing == ["model.norm.weight"] and e.value.unexpected == [extra]


def test_model_spec_rejects_bad_schedules():
    arch, cfg, _ = resolve(TINY_A["config"])
    spec = arch.build_spec(cfg)
    kw = {f: getattr(spec, f) for f in spec.__dataclass_fields__}
    ModelSpec(**dict(kw, schedule=[LayerRun(0), LayerRun(1), LayerRun(0), LayerRun(1, cache_of=1)]))  # fine
    with pytest.raises(ValueError, match="names layer 2"):
        ModelSpec(**dict(kw, schedule=[LayerRun(0), LayerRun(2)]))
    with pytest.raises(ValueError, match="not earlier"):
        ModelSpec(**dict(kw, schedule=[LayerRun(0, cache_of=1), LayerRun(1)]))
    with pytest.raises(ValueError, match="no cache of its own"):
        ModelSpec(**dict(kw, schedule=[LayerRun(0), LayerRun(1, cache_of=0), LayerRun(0, cache_of=1)]))


def test_command_line_keeps_the_reference_option_names(tmp_path, monkeypatch):
    """jllm/server.py:245-269: --model-path (env JLLM_MODEL_PATH), --max-num-seqs 4,
    --max-model-len 2048, --max-prefill-len 512, --dtype {bf16,fp32} default bf16."""
    from jax_vllm_amd.engine import cli

    monkeypatch.setenv("JLLM_MODEL_PATH", "/some/where")
    a = cli.build_parser().parse_args([])
    assert (a.model_path, a.max_num_seqs, a.max_model_len, a.max_prefill_len, a.dtype) == ("/some/where", 4, 2048, 512, "bf16")
    assert cli.parse_ids("1, 2 3") == [1, 2, 3]
    (tmp_path / "p.txt").write_text("5 6 7\n\n8,9\n")
    (tmp_path / "p.json").write_text("[[1, 2], [3]]")
    assert cli.read_prompts(cli.build_parser().parse_args(["--prompt-ids", "4 4", "--prompt-file", str(tmp_path / "p.txt")])) == [[4, 4], [5, 6, 7], [8, 9]]
    assert cli.read_prompts(cli.build_parser().parse_args(["--prompt-file", str(tmp_path / "p.json")])) == [[1, 2], [3]]
    # the random-weights mode writes a loadable folder without a GPU
    (tmp_path / "c.json").write_text(json.dumps(TINY_A["config"]))
    assert cli.main(["--random-config", str(tmp_path / "c.json"), "--random-seed", "3", "--write-model", str(tmp_path / "m")]) == 0
    assert (tmp_path / "m" / "config.json").exists() and (tmp_path / "m" / "model.safetensors").exists()
    assert cli.main([]) == 2
