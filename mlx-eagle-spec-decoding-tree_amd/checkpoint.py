"""Reader for MLX-community 4-bit checkpoints on local disk (mlx_utils.py:59-136).

A checkpoint directory holds `config.json` and one or more `model*.safetensors` shards
(`weight*.safetensors` in older exports).  Quantised linears and the embedding are stored as
`<name>.weight` (uint32, eight nibbles per word), `<name>.scales`, `<name>.biases` and an
optional dense `<name>.bias`; `config["quantization"]` gives `group_size` and `bits`.

Only local paths are read; nothing is downloaded.  safetensors files are opened with
`safetensors.safe_open`, which executes nothing from the file.
"""
import glob
import json
import os

import torch

from .synth import ModelArgs

_ARG_FIELDS = set(ModelArgs.__dataclass_fields__)


def load_config(model_path):
    path = os.path.join(str(model_path), "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"config.json not found in {model_path}")
    with open(path) as f:
        return json.load(f)


def model_args_from_config(config):
    """ModelArgs from a config dict: unknown keys are ignored (ModelArgs.from_dict of the
    reference), qwen2 models have biases on q/k/v (mlx_utils.py:120-121), and the quantisation
    has to be the one the kernels implement."""
    q = config.get("quantization")
    if q is None:
        raise ValueError("the checkpoint is not quantised: config.json has no 'quantization' entry")
    if int(q.get("group_size", 0)) != 64 or int(q.get("bits", 0)) != 4:
        raise ValueError(f"only group_size=64, bits=4 checkpoints are supported, got {q}")
    fields = {k: v for k, v in config.items() if k in _ARG_FIELDS}
    args = ModelArgs(**fields)
    if config.get("model_type") == "qwen2":
        args.attention_bias = True
    args.group_size, args.bits = 64, 4
    return args


def weight_files(model_path):
    files = sorted(glob.glob(os.path.join(str(model_path), "model*.safetensors")))
    if not files:   # older exports (mlx_utils.py:93-95)
        files = sorted(glob.glob(os.path.join(str(model_path), "weight*.safetensors")))
    if not files:
        raise FileNotFoundError(f"No safetensors found in {model_path}")
    return files


def sanitize(weights):
    """Drop precomputed rotary tables (mlx_llama.py:315-319)."""
    return {k: v for k, v in weights.items() if "self_attn.rotary_emb.inv_freq" not in k}


def load_weights(model_path, device="cpu"):
    """All tensors of every shard as a flat dict of torch tensors on `device`.  Packed uint32
    words are kept bit for bit (as int32 storage); floating-point tensors that are not fp16
    (bf16 exports) are converted to fp16, the type the kernels compute in; a value that does not
    fit fp16 raises ValueError."""
    from safetensors import safe_open

    out = {}
    for wf in weight_files(model_path):
        with safe_open(wf, framework="pt", device="cpu") as f:
            for key in f.keys():
                t = f.get_tensor(key)
                if t.dtype == torch.uint32:
                    t = t.view(torch.int32)
                elif t.dtype.is_floating_point and t.dtype != torch.float16:
                    wide = t
                    t = wide.to(torch.float16)
                    # bf16 / fp32 reach beyond fp16's range: refuse rather than carry inf
                    if bool((torch.isinf(t) & ~torch.isinf(wide)).any()):
                        raise ValueError(f"{key} ({wide.dtype}) holds values beyond the fp16 range; "
                                         "the kernels compute in fp16")
                out[key] = t.contiguous().to(device)
    return sanitize(out)


def check_quantized(args, weights):
    """Every linear of the decoder has to be quantised (legacy exports with dense layers,
    mlx_utils.py:127-131, are not supported) and shaped as the config says."""
    D, I, V = args.hidden_size, args.intermediate_size, args.vocab_size
    H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
    want = {"self_attn.q_proj": (H * hd, D), "self_attn.k_proj": (G * hd, D),
            "self_attn.v_proj": (G * hd, D), "self_attn.o_proj": (D, H * hd),
            "mlp.gate_proj": (I, D), "mlp.up_proj": (I, D), "mlp.down_proj": (D, I)}
    names = {"model.embed_tokens": (V, D)}
    if not args.tie_word_embeddings:
        names["lm_head"] = (V, D)
    for i in range(args.num_hidden_layers):
        for k, shp in want.items():
            names[f"model.layers.{i}.{k}"] = shp
    for name, (n, k) in names.items():
        for part, shape in (("weight", (n, k // 8)), ("scales", (n, k // 64)), ("biases", (n, k // 64))):
            t = weights.get(f"{name}.{part}")
            if t is None:
                raise ValueError(f"{name}.{part} is missing: the layer is not quantised")
            if tuple(t.shape) != shape:
                raise ValueError(f"{name}.{part} has shape {tuple(t.shape)}, expected {shape}")
        if weights[f"{name}.weight"].dtype not in (torch.int32, torch.uint32):
            raise ValueError(f"{name}.weight is not packed uint32")


def load_model(model_path, device, model_config=None):
    """`load_model(model_path)` of the reference (mlx_utils.py:59-136) for a local directory:
    returns (Model, config)."""
    from . import llama

    config = load_config(model_path)
    config.update(model_config or {})
    args = model_args_from_config(config)
    weights = load_weights(model_path, device)
    check_quantized(args, weights)
    return llama.Model(args, weights, device), config
