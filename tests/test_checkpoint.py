"""Reader for MLX-community 4-bit checkpoint directories (mlx_utils.py:59-136): a tiny synthetic
checkpoint is written with safetensors in the on-disk layout (uint32 packed weights, fp16 or
bf16 scales/biases, sharded files, config.json with a quantization entry) and read back."""
import json
import os

import numpy as np
import pytest
import torch

from mlx_eagle_spec_decoding_tree_amd import checkpoint, synth

save_file = pytest.importorskip("safetensors.numpy").save_file


def config_of(args, **extra):
    cfg = {"model_type": args.model_type, "hidden_size": args.hidden_size,
           "num_hidden_layers": args.num_hidden_layers, "intermediate_size": args.intermediate_size,
           "num_attention_heads": args.num_attention_heads,
           "num_key_value_heads": args.num_key_value_heads, "head_dim": args.head_dim,
           "rms_norm_eps": args.rms_norm_eps, "vocab_size": args.vocab_size,
           "rope_theta": args.rope_theta, "tie_word_embeddings": args.tie_word_embeddings,
           "quantization": {"group_size": 64, "bits": 4},
           # keys the reader has to ignore
           "architectures": ["Qwen2ForCausalLM"], "torch_dtype": "float16", "use_cache": True}
    cfg.update(extra)
    return cfg


def write_checkpoint(path, args, weights, shards=2, prefix="model", cfg=None):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg if cfg is not None else config_of(args), f)
    keys = sorted(weights)
    for i in range(shards):
        part = {k: weights[k] for k in keys[i::shards]}
        name = f"{prefix}.safetensors" if shards == 1 else f"{prefix}-{i + 1:05d}-of-{shards:05d}.safetensors"
        save_file(part, os.path.join(path, name))


@pytest.fixture
def tiny():
    args = synth.tiny()
    return args, synth.make_model_weights(args, seed=5)


def test_round_trip_sharded(tmp_path, tiny):
    args, weights = tiny
    write_checkpoint(tmp_path, args, weights, shards=3)
    got = checkpoint.load_weights(tmp_path)
    assert set(got) == set(weights)
    for k, v in weights.items():
        t = got[k]
        if v.dtype == np.uint32:
            assert t.dtype == torch.int32
            assert np.array_equal(t.numpy().view(np.uint32), v), k
        else:
            assert t.dtype == torch.float16
            assert np.array_equal(t.numpy(), v), k


def test_config_to_model_args(tmp_path, tiny):
    args, weights = tiny
    write_checkpoint(tmp_path, args, weights)
    cfg = checkpoint.load_config(tmp_path)
    got = checkpoint.model_args_from_config(cfg)
    assert got == args
    # a qwen2 config does not say attention_bias; the loader sets it (mlx_utils.py:120-121)
    assert "attention_bias" not in cfg and got.attention_bias is True
    llama_cfg = dict(cfg, model_type="llama")
    assert checkpoint.model_args_from_config(llama_cfg).attention_bias is False
    checkpoint.check_quantized(got, checkpoint.load_weights(tmp_path))


def test_old_shard_names_and_missing_files(tmp_path, tiny):
    args, weights = tiny
    write_checkpoint(tmp_path / "old", args, weights, shards=1, prefix="weights")
    assert set(checkpoint.load_weights(tmp_path / "old")) == set(weights)
    os.makedirs(tmp_path / "empty")
    with pytest.raises(FileNotFoundError, match="No safetensors found"):
        checkpoint.load_weights(tmp_path / "empty")
    with pytest.raises(FileNotFoundError, match="config.json"):
        checkpoint.load_config(tmp_path / "empty")


def test_rotary_tables_dropped_and_bf16_converted(tmp_path, tiny):
    args, weights = tiny
    main = {k: v for k, v in weights.items() if k != "model.norm.weight"}
    write_checkpoint(tmp_path, args, main, shards=1)
    extra = {"model.layers.0.self_attn.rotary_emb.inv_freq": torch.ones(32),
             "model.norm.weight": torch.from_numpy(weights["model.norm.weight"]).to(torch.bfloat16)}
    from safetensors.torch import save_file as save_torch
    save_torch(extra, str(tmp_path / "model-extra.safetensors"))
    got = checkpoint.load_weights(tmp_path)
    assert not any("rotary_emb" in k for k in got)
    nw = got["model.norm.weight"]
    assert nw.dtype == torch.float16
    assert torch.equal(nw, extra["model.norm.weight"].to(torch.float16))


@pytest.mark.parametrize("quant", [None, {"group_size": 32, "bits": 4}, {"group_size": 64, "bits": 8}])
def test_unsupported_quantisation_is_refused(tiny, quant):
    args, _ = tiny
    cfg = config_of(args)
    if quant is None:
        del cfg["quantization"]
    else:
        cfg["quantization"] = quant
    with pytest.raises(ValueError):
        checkpoint.model_args_from_config(cfg)


def test_dense_or_misshapen_layer_is_refused(tmp_path, tiny):
    args, weights = tiny
    w = dict(weights)
    del w["model.layers.1.mlp.up_proj.scales"]
    write_checkpoint(tmp_path / "a", args, w)
    with pytest.raises(ValueError, match="up_proj.scales"):
        checkpoint.check_quantized(args, checkpoint.load_weights(tmp_path / "a"))
    w = dict(weights)
    w["lm_head.weight"] = w["lm_head.weight"][:, :-1].copy()
    write_checkpoint(tmp_path / "b", args, w)
    with pytest.raises(ValueError, match="lm_head.weight has shape"):
        checkpoint.check_quantized(args, checkpoint.load_weights(tmp_path / "b"))


def test_rope_scaling_is_validated(tiny):
    args, _ = tiny
    with pytest.raises(ValueError, match="factor"):
        checkpoint.model_args_from_config(config_of(args, rope_scaling={"type": "linear"}))
    got = checkpoint.model_args_from_config(
        config_of(args, rope_scaling={"rope_type": "linear", "factor": 2.0}))
    assert got.rope_scaling["factor"] == 2.0


@pytest.mark.gpu
def test_loaded_model_matches_in_memory_model(tmp_path, tiny):
    """The model read from disk gives the same tree-decoding logits, bit for bit, as the model
    built from the same arrays in memory."""
    from mlx_eagle_spec_decoding_tree_amd import eagle, llama
    from mlx_eagle_spec_decoding_tree_amd.cache import make_prompt_cache
    from oracle import tree_oracle
    from util import to_dev

    args, weights = tiny
    write_checkpoint(tmp_path, args, weights, shards=2)
    dev = torch.device("cuda:0")
    loaded, cfg = checkpoint.load_model(tmp_path, dev)
    assert cfg["quantization"] == {"group_size": 64, "bits": 4}
    direct = llama.Model.from_numpy(args, weights, dev)
    P, T = 40, 16
    rng = np.random.default_rng(1)
    G, hd = args.num_key_value_heads, args.head_dim
    prefix = [(rng.normal(size=(G, P, hd)).astype(np.float16), rng.normal(size=(G, P, hd)).astype(np.float16))
              for _ in range(args.num_hidden_layers)]
    parents = synth.random_tree(rng, T)
    depth, anc = tree_oracle.tree_from_parents(parents)
    tokens = rng.integers(0, args.vocab_size, T).astype(np.int32)
    tree_mask = to_dev(tree_oracle.additive_mask(anc), dev).to(torch.bfloat16)
    outs = []
    for m in (loaded, direct):
        assert m.args == args
        cache = make_prompt_cache(m, capacity=P + T + 16)
        for c, (k, v) in zip(cache, prefix):
            c.keys[0, :, :P].copy_(to_dev(k, dev)); c.values[0, :, :P].copy_(to_dev(v, dev))
            c.offset = P
        cache[0].sync_len()
        logits = eagle.tree_decoding(to_dev(tokens[None], dev), tree_mask, to_dev(depth, dev), m, cache)[0]
        outs.append(logits.float().cpu())
    assert torch.isfinite(outs[0]).all()
    assert torch.equal(outs[0], outs[1])


def test_bf16_values_beyond_fp16_are_refused(tmp_path, tiny):
    """bf16 exports are converted to fp16; a scale that fp16 cannot hold must not become inf
    silently."""
    from safetensors.torch import save_file as save_torch

    args, weights = tiny
    with open(os.path.join(tmp_path, "config.json"), "w") as f:
        json.dump(config_of(args), f)
    tw = {}
    for k, v in weights.items():
        t = torch.from_numpy(v.view(np.int32) if v.dtype == np.uint32 else v)
        tw[k] = t.to(torch.bfloat16) if t.dtype == torch.float16 else t
    save_torch(tw, os.path.join(tmp_path, "model.safetensors"))
    got = checkpoint.load_weights(tmp_path)
    assert got["model.norm.weight"].dtype == torch.float16
    bad = dict(tw)
    bad["model.norm.weight"] = tw["model.norm.weight"].clone()
    bad["model.norm.weight"][3] = 1e5
    save_torch(bad, os.path.join(tmp_path, "model.safetensors"))
    with pytest.raises(ValueError, match="fp16 range"):
        checkpoint.load_weights(tmp_path)


LLAMA3_SCALING = {"factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                  "original_max_position_embeddings": 8192, "rope_type": "llama3"}


def test_llama32_style_config_loads_with_the_llama3_table(tmp_path):
    """The configuration of the model the reference's own test loads
    (mlx_eagle_tests.py:19: Llama-3.2-1B): rope_scaling of type llama3, tied head, head_dim 64."""
    args = synth.ModelArgs(model_type="llama", hidden_size=256, num_hidden_layers=1,
                           intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                           head_dim=64, vocab_size=512, rms_norm_eps=1e-5, rope_theta=5e5,
                           attention_bias=False, tie_word_embeddings=True,
                           max_position_embeddings=131072, rope_scaling=dict(LLAMA3_SCALING))
    weights = synth.make_model_weights(args, seed=3)
    cfg = config_of(args, rope_scaling=dict(LLAMA3_SCALING), max_position_embeddings=131072,
                    architectures=["LlamaForCausalLM"])
    write_checkpoint(tmp_path, args, weights, shards=1, cfg=cfg)
    got = checkpoint.model_args_from_config(checkpoint.load_config(tmp_path))
    assert got.rope_scaling == LLAMA3_SCALING and got.max_position_embeddings == 131072
    inv, scale = synth.inv_freqs(got)
    plain, _ = synth.inv_freqs(synth.ModelArgs(model_type="llama", hidden_size=256, num_attention_heads=4,
                                               head_dim=64, rope_theta=5e5))
    assert scale == 1.0 and inv.shape == (32,) and inv.dtype == np.float32
    assert np.array_equal(inv[:8], plain[:8])                    # short wavelengths untouched
    assert np.allclose(inv[-4:], plain[-4:] / 32.0, rtol=1e-6)   # long ones slowed by `factor`
    model, _ = checkpoint.load_model(tmp_path, "cpu")
    assert np.array_equal(model.model.layers[0].self_attn._inv_freqs.numpy(), inv)
