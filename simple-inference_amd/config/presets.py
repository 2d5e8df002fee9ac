"""Named config.json dictionaries: data, not code paths.

These are the shapes that the measurement program and the command line can
build random weights for.  Each is the dictionary a config.json of that model
would hold, and goes through the same ``parse_config`` as a file does.  The
reference has one preset, ``ModelConfig.llama_3_2_3b`` (``config.py:111-135``).
"""

from __future__ import annotations

import copy

_LLAMA3_SCALING_32 = {
    "rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
    "high_freq_factor": 4.0, "original_max_position_embeddings": 8192,
}

def _feduzen_layer(ff, weights_of=None):
    layer = {"type": "attention", "mlp": {"kind": "dense", "ff": ff} if ff else None,
             "mixer": {"heads": 8, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.11, "mask": {"size": 256},
                       "rot": {"dims": 32, "base": 100000.0,
                               "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 1024}}}}
    if weights_of is not None:
        layer["weights_of"] = weights_of
    return layer


_FAMEPEL_LATENT = {"type": "latent_attention",
                   "mixer": {"dim": 64, "heads": 8, "kv_rank": 96, "q_rank": 192, "rot_dim": 32, "vdim": 64, "scale": 0.1,
                             "rot": {"base": 10000.0, "dims": 32,
                                     "scaling": {"factor": 4.0, "original": 2048, "fast": 32.0, "slow": 1.0}}}}


def _famepel_layer(mixer):
    return dict(mixer, mlp={"kind": "moe", "expert": {"ff": 256},
                            "router": {"experts": 8, "top": 2, "scale": 2.0, "groups": {"count": 4, "keep": 2}}})


def _tadinex_layer(kind, mlp):
    if kind == "delta":
        mixer = {"conv": 4, "dim": 64, "heads": 8, "kv_heads": 4, "vdim": 64}
    else:
        mixer = {"left": {"dim": 64, "vdim": 64, "heads": 8, "kv_heads": 2, "mask": {"size": 128}, "scale": 0.125,
                          "rot": {"base": 100000.0, "dims": 32,
                                  "scaling": {"factor": 4.0, "original": 1024, "fast": 32.0, "slow": 1.0}}},
                 "left_scale": 0.7, "right": {"dim": 64, "vdim": 64, "heads": 4, "decay": [0.75, 0.9, 0.97, 0.995]},
                 "right_scale": 0.9}
    return {"type": kind, "mixer": mixer, "mlp": mlp}


_TADINEX_EXPERTS = {"kind": "moe", "router": {"experts": 8, "identity": 2, "top": 2}, "expert": {"ff": 256, "limit": 7.0},
                    "shared": {"ff": 512, "limit": 7.0}}


def _mogisun_layer(kind, moe):
    if kind == "attention":
        mixer = {"heads": 8, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.125, "q_temp": {"coef": 0.2, "every": 512}}
    else:
        mixer = {"heads": 8, "dim": 64, "vdim": 64, "tau": 8.0, "rank": 32}
    mlp = {"kind": "dense", "ff": 1536}
    if moe:
        mlp = {"kind": "moe", "router": {"experts": 16, "top": 2}, "expert": {"ff": 384}, "shared": {"ff": 512}}
    return {"type": kind, "mixer": mixer, "mlp": mlp}


PRESETS = {
    "llama-3.2-3b": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": 3072, "intermediate_size": 8192, "num_hidden_layers": 28,
        "vocab_size": 128256, "num_attention_heads": 24, "num_key_value_heads": 8, "head_dim": 128,
        "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "rope_scaling": _LLAMA3_SCALING_32,
        "max_position_embeddings": 131072, "bos_token_id": 128000, "eos_token_id": 128001,
        "tie_word_embeddings": True, "torch_dtype": "bfloat16", "hidden_act": "silu",
    },
    "llama-3.2-1b": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": 2048, "intermediate_size": 8192, "num_hidden_layers": 16,
        "vocab_size": 128256, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
        "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "rope_scaling": _LLAMA3_SCALING_32,
        "max_position_embeddings": 131072, "bos_token_id": 128000, "eos_token_id": 128001,
        "tie_word_embeddings": True, "torch_dtype": "bfloat16", "hidden_act": "silu",
    },
    "llama-3.1-8b": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": 4096, "intermediate_size": 14336, "num_hidden_layers": 32,
        "vocab_size": 128256, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
        "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
        "rope_scaling": dict(_LLAMA3_SCALING_32, factor=8.0),
        "max_position_embeddings": 131072, "bos_token_id": 128000, "eos_token_id": 128001,
        "tie_word_embeddings": False, "torch_dtype": "bfloat16", "hidden_act": "silu",
    },
    # a small model of the Feduzen design: five runs of three layers' weights, one layer without a feed-forward
    "feduzen-small": {
        "architecture": "Feduzen", "vocab": 4096, "width": 512, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-6},
        "layers": [_feduzen_layer(1536), _feduzen_layer(None), _feduzen_layer(None, weights_of=1),
                   _feduzen_layer(1536), _feduzen_layer(1536, weights_of=0)],
    },
    # a small model of the Mogisun design: softmax and linear attention in turn, dense and routed feed-forwards, the
    # middle four layers walked twice
    "mogisun-small": {
        "architecture": "Mogisun", "vocab": 4096, "width": 512, "norm": {"eps": 1e-6}, "logit_scale": 1.5,
        "logit_softcap": 30.0, "loop": {"start": 1, "stop": 5, "times": 2},
        "layers": [_mogisun_layer("attention", False), _mogisun_layer("gla", True), _mogisun_layer("attention", False),
                   _mogisun_layer("gla", True), _mogisun_layer("attention", False), _mogisun_layer("gla", True)],
    },
    # a small model of the Famepel design: its three mixers in turn, the last layer reading the third's latent, grouped
    # experts
    "famepel-small": {
        "architecture": "Famepel", "vocab": 4096, "width": 512, "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
        "layers": [_famepel_layer({"type": "mamba2", "mixer": {"conv": 4, "groups": 2, "heads": 8, "norm_groups": 2,
                                                                 "state": 64, "vdim": 64}}),
                   _famepel_layer({"type": "hgrn2", "mixer": {"dim": 64, "heads": 8, "vdim": 64}}),
                   _famepel_layer(_FAMEPEL_LATENT),
                   _famepel_layer({"type": "mamba2", "mixer": {"conv": 4, "groups": 2, "heads": 8, "norm_groups": 2,
                                                                 "state": 64, "vdim": 64}}),
                   _famepel_layer(dict(_FAMEPEL_LATENT, mixer=dict(_FAMEPEL_LATENT["mixer"], kv_from=2)))],
    },
    # a small model of the Tadinex design: three delta-rule layers after every layer of the two mixers side by side,
    # a dense feed-forward first, routed experts after it
    "tadinex-small": {
        "architecture": "Tadinex", "vocab": 4096, "width": 512, "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
        "residual_mult": 0.8,
        "layers": [_tadinex_layer("parallel", {"kind": "dense", "ff": 1536}), _tadinex_layer("delta", _TADINEX_EXPERTS),
                   _tadinex_layer("delta", _TADINEX_EXPERTS), _tadinex_layer("delta", _TADINEX_EXPERTS),
                   _tadinex_layer("parallel", _TADINEX_EXPERTS), _tadinex_layer("delta", _TADINEX_EXPERTS)],
    },
    "tiny-a": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": 64, "intermediate_size": 128, "num_hidden_layers": 2,
        "vocab_size": 256, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
        "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "rope_scaling": None,
        "max_position_embeddings": 2048, "bos_token_id": 1, "eos_token_id": 2,
        "tie_word_embeddings": True, "torch_dtype": "bfloat16", "hidden_act": "silu",
    },
    "tiny-b": {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": 96, "intermediate_size": 224, "num_hidden_layers": 3,
        "vocab_size": 384, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
        "rms_norm_eps": 1e-6, "rope_theta": 500000.0,
        "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                         "high_freq_factor": 4.0, "original_max_position_embeddings": 64},
        "max_position_embeddings": 4096, "bos_token_id": 1, "eos_token_id": 2,
        "tie_word_embeddings": False, "torch_dtype": "bfloat16", "hidden_act": "silu",
    },
}


def preset(name: str) -> dict:
    try:
        return copy.deepcopy(PRESETS[name])
    except KeyError:
        raise KeyError(f"unknown preset {name!r}; known: {', '.join(sorted(PRESETS))}") from None
