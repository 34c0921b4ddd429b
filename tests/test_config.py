"""The typed configuration, the registry and the engine configuration."""

import json

import pytest

from atom_amd.config import (Config, ConfigError, Qwen3Config, build_model, known_architectures,
                             model_config_from_dict, register_architecture, unregister_architecture)
from atom_amd.engine.arg_utils import EngineArgs, FlexibleArgumentParser
from atom_amd.sampling import SamplingParams
from tiny import TINY_A, TINY_B, TINY_C


def test_reads_every_size_from_config_json():
    a, b, c = (model_config_from_dict(x) for x in (TINY_A, TINY_B, TINY_C))
    assert (a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (64, 4, 2, 16)
    assert (b.hidden_size, b.num_attention_heads * b.head_dim, b.vocab_size, b.rms_norm_eps) == (96, 192, 311, 1e-5)
    assert a.tie_word_embeddings and not b.tie_word_embeddings
    assert c.attention_bias and c.window_of_layer(1) == 40 and c.window_of_layer(0) is None
    assert model_config_from_dict({**TINY_C, "use_sliding_window": False}).window_of_layer(1) is None


def test_fallbacks_follow_the_reference():
    raw = {k: v for k, v in TINY_A.items() if k not in ("head_dim", "max_position_embeddings", "rope_theta")}
    raw["rope_parameters"] = {"rope_theta": 12345.0, "rope_type": "default"}
    cfg = model_config_from_dict(raw)
    assert cfg.head_dim == 64 // 4            # hidden_size // heads
    assert cfg.max_position_embeddings == 8192
    assert cfg.rope_theta == 12345.0
    assert isinstance(model_config_from_dict({**TINY_A, "rope_theta": 10000}).rope_theta, float)


def test_round_trip(tmp_path):
    cfg = model_config_from_dict(TINY_C)
    cfg.save(str(tmp_path))
    with open(tmp_path / "config.json") as f:
        again = model_config_from_dict(json.load(f))
    assert again == cfg


@pytest.mark.parametrize("change,needle", [
    ({"num_key_value_heads": 3}, "multiple"), ({"hidden_act": "gelu"}, "silu"), ({"head_dim": 15}, "even"),
    ({"vocab_size": 0}, "positive"), ({"rope_scaling": {"rope_type": "yarn", "factor": 4}}, "yarn"),
    ({"hidden_size": "64"}, "int"), ({"architectures": ["NoSuchModel"]}, "NoSuchModel"),
    ({"layer_types": ["full_attention"]}, "layer_types"),
])
def test_bad_configs_are_refused(change, needle):
    with pytest.raises(ConfigError) as e:
        model_config_from_dict({**TINY_A, **change})
    assert needle in str(e.value)


def test_missing_key_is_named():
    raw = dict(TINY_A)
    del raw["intermediate_size"]
    with pytest.raises(ConfigError, match="intermediate_size"):
        model_config_from_dict(raw)


def test_registry_lists_known_and_takes_new():
    assert "Qwen3ForCausalLM" in known_architectures()
    with pytest.raises(ConfigError) as e:
        model_config_from_dict({**TINY_A, "architectures": ["Mystery"]})
    assert "Qwen3ForCausalLM" in str(e.value)
    from atom_amd.models.qwen3 import qwen3_spec
    register_architecture("AliasForCausalLM", Qwen3Config, qwen3_spec)
    try:
        model = build_model(model_config_from_dict({**TINY_A, "architectures": ["AliasForCausalLM"]}))
        assert len(model.blocks) == 2
        with pytest.raises(KeyError):
            register_architecture("AliasForCausalLM", Qwen3Config, qwen3_spec)
    finally:
        unregister_architecture("AliasForCausalLM")


def test_model_is_assembled_from_the_configuration():
    model = build_model(model_config_from_dict(TINY_C))
    assert [b.mixer.window for b in model.blocks] == [None, 40, 40, None]
    assert model.blocks[0].mixer.qkv_bias and model.blocks[0].mixer.num_kv_heads == 2
    assert model.blocks[2].ffn.intermediate_size == 200 and model.final_norm.eps == 3e-6
    assert model.head.tied_to is None
    assert build_model(model_config_from_dict(TINY_A)).head.tied_to is not None


def test_engine_config(tmp_path):
    mc = model_config_from_dict({**TINY_B, "eos_token_id": [7, 9]})
    cfg = Config("x", model_config=mc, max_model_len=100000, dtype="fp32")
    assert cfg.max_model_len == 256 and cfg.dtype == "float32"
    assert cfg.eos_token_id == 7 and cfg.stop_token_ids == [9]
    with pytest.raises(ConfigError):
        Config("x", model_config=mc, dtype="fp8")
    with pytest.raises(ConfigError):
        Config("x", model_config=mc, kv_cache_block_size=0)
    with pytest.raises(ConfigError):
        Config("x", model_config=mc, long_prefill_token_threshold=4)
    with pytest.raises(ConfigError):
        Config(str(tmp_path))   # no config.json there
    mc.save(str(tmp_path))
    assert Config(str(tmp_path), hf_overrides={"rms_norm_eps": 1e-3}).model_config.rms_norm_eps == 1e-3


def test_sampling_params_defaults_and_checks():
    sp = SamplingParams()
    assert (sp.temperature, sp.top_k, sp.top_p, sp.max_tokens, sp.ignore_eos, sp.n) == (1.0, -1, 1.0, 64, False, 1)
    for bad in (dict(top_k=0), dict(top_k=-2), dict(top_p=0.0), dict(top_p=1.1), dict(n=0), dict(temperature=-1.0)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)


def test_cli_flags_in_both_spellings():
    parser = FlexibleArgumentParser()
    EngineArgs.add_cli_args(parser)
    a = EngineArgs.from_cli_args(parser.parse_args(["--model", "m", "--max-model-len", "99", "--block_size=32",
                                                    "--no-enable-chunked-prefill", "--max_num_seqs", "7",
                                                    "--mark-trace"]))
    assert (a.model, a.max_model_len, a.block_size, a.enable_chunked_prefill, a.max_num_seqs) == ("m", 99, 32, False, 7)
    assert a.mark_trace and not EngineArgs(model="m").mark_trace
    b = EngineArgs.from_cli_args(parser.parse_args(["--model", "m", "--level", "0", "--cudagraph-mode", "NONE"]))
    assert b._get_engine_kwargs()["enforce_eager"] and "level" not in b._get_engine_kwargs()
    assert not a._get_engine_kwargs()["enforce_eager"]
    kw = a._get_engine_kwargs()
    assert kw["kv_cache_block_size"] == 32 and "block_size" not in kw
    assert kw["cudagraph_capture_sizes"][:3] == [1, 2, 4]


def test_cli_graph_sizes_for_steps_with_prompt_portions():
    parser = FlexibleArgumentParser()
    EngineArgs.add_cli_args(parser)
    off = EngineArgs.from_cli_args(parser.parse_args(["--model", "m"]))._get_engine_kwargs()
    on = EngineArgs.from_cli_args(parser.parse_args(["--model", "m", "--cudagraph-prefill-sizes", "[256, 512]"]))
    assert off["cudagraph_prefill_sizes"] == [] and on._get_engine_kwargs()["cudagraph_prefill_sizes"] == [256, 512]


def test_cli_renders_prompts_through_the_chat_template(tmp_path):
    """With a tokenizer that has a chat template the command line sends one user message with the generation
    prompt appended (atom/examples/simple_inference.py:66-70); without a template, the text itself."""
    from tokenizers import Tokenizer, models, pre_tokenizers
    from transformers import PreTrainedTokenizerFast

    from atom_amd.examples.simple_inference import render_chat

    words = ["<|im_start|>", "<|im_end|>", "user", "assistant", "1+2+3=?", "[UNK]"]
    raw = Tokenizer(models.WordLevel({w: i for i, w in enumerate(words)}, unk_token="[UNK]"))
    raw.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok = PreTrainedTokenizerFast(tokenizer_object=raw, unk_token="[UNK]")
    assert render_chat(tok, "1+2+3=?") == "1+2+3=?"
    tok.chat_template = ("{% for m in messages %}<|im_start|> {{ m['role'] }} {{ m['content'] }} <|im_end|> {% endfor %}"
                         "{% if add_generation_prompt %}<|im_start|> assistant{% endif %}")
    text = render_chat(tok, "1+2+3=?")
    assert text == "<|im_start|> user 1+2+3=? <|im_end|> <|im_start|> assistant"
    assert tok.encode(text) == [0, 2, 4, 1, 0, 3]


def test_profile_offline_arguments():
    """The offline profiling command takes the engine's flags and its own four with the reference's defaults
    (atom/examples/profile_offline.py:19-41), and its prompt is --input-length seeded ids when random."""
    from types import SimpleNamespace

    from atom_amd.examples import profile_offline as po

    args = po.parser.parse_args(["--model", "m"])
    assert (args.input_length, args.output_length, args.bs, args.random_input) == (128, 32, 1, False)
    assert args.torch_profiler_dir is None and po.DEFAULT_TRACE_DIR == "./profiler_traces"
    args = po.parser.parse_args(["--model", "m", "--input_length", "9", "--bs=4", "--random-input", "--seed", "5"])
    llm = SimpleNamespace(tokenizer=None, config=SimpleNamespace(model_config=SimpleNamespace(vocab_size=50)))
    ids = po.make_prompt(llm, args)
    assert len(ids) == 9 and all(0 <= t < 50 for t in ids) and ids == po.make_prompt(llm, args)
    args.random_input = False
    assert po.make_prompt(SimpleNamespace(tokenizer=object(), config=llm.config), args) == po.FIXED_PROMPT
    with pytest.raises(SystemExit):
        po.main(["--model", "m", "--bs", "0"])
