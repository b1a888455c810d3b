"""Local checkpoint reader: HuggingFace BigBird / BERT weight names -> this package's layer weights.

The reference builds its layers from a live HuggingFace module (`from_torch`,
python/modeling_bert.py:62-69, :84-91, :107-113, :137-163); this reads the same tensors from a
checkpoint on disk (`model.safetensors` or `pytorch_model.bin`, with `config.json` beside it when
present) and applies the same re-layout: Q | K | V weights concatenated and transposed to
`[in, out]`, every dense weight transposed to `[in, out]`.  Nothing is downloaded and nothing is
executed from the file: safetensors, or `torch.load(..., weights_only=True)`.

This module imports neither the HIP library nor the extension, so the mapping can be checked on a
machine without a GPU; `modeling_bert.BertModelNoPooler.from_local_checkpoint` is the caller.
"""
import json
import os
import re

import torch

EMBEDDING_KEYS = ("word_embeddings.weight", "position_embeddings.weight", "token_type_embeddings.weight",
                  "LayerNorm.weight", "LayerNorm.bias")
_LAYER_KEYS = (
    "attention.self.query.weight", "attention.self.query.bias", "attention.self.key.weight",
    "attention.self.key.bias", "attention.self.value.weight", "attention.self.value.bias",
    "attention.output.dense.weight", "attention.output.dense.bias", "attention.output.LayerNorm.weight",
    "attention.output.LayerNorm.bias", "intermediate.dense.weight", "intermediate.dense.bias",
    "output.dense.weight", "output.dense.bias", "output.LayerNorm.weight", "output.LayerNorm.bias")


def read_state_dict(path):
    """`path`: a checkpoint file, or a directory holding `model.safetensors` / `pytorch_model.bin`.
    Returns (state_dict on the CPU, config dict or {})."""
    cfg = {}
    if os.path.isdir(path):
        cfg_path = os.path.join(path, "config.json")
        if os.path.exists(cfg_path):
            with open(cfg_path) as f:
                cfg = json.load(f)
        for name in ("model.safetensors", "pytorch_model.bin"):
            if os.path.exists(os.path.join(path, name)):
                path = os.path.join(path, name)
                break
        else:
            raise FileNotFoundError("no model.safetensors or pytorch_model.bin in %s" % path)
    if path.endswith(".safetensors"):
        from safetensors.torch import load_file
        return load_file(path, device="cpu"), cfg
    sd = torch.load(path, map_location="cpu", weights_only=True)
    if not isinstance(sd, dict):
        raise ValueError("%s does not hold a state dict" % path)
    return sd, cfg


def _strip_prefix(sd):
    """Task heads nest the encoder under `bert.` (BigBirdFor...), `bigbird.` or `model.`."""
    for prefix in ("", "bert.", "bigbird.", "model.", "big_bird."):
        if prefix + "embeddings.word_embeddings.weight" in sd:
            return {k[len(prefix):]: v for k, v in sd.items() if k.startswith(prefix)}
    raise KeyError("no `embeddings.word_embeddings.weight` in the checkpoint (known prefixes: bert., bigbird., model.)")


def convert_state_dict(sd):
    """-> (embeddings: dict of the five tensors under EMBEDDING_KEYS,
           layers: list of dicts with the keys of `modeling_bert.random_layer_weights`)."""
    sd = _strip_prefix(sd)
    missing = [k for k in EMBEDDING_KEYS if "embeddings." + k not in sd]
    if missing:
        raise KeyError("checkpoint lacks embeddings.%s" % missing[0])
    emb = {k: sd["embeddings." + k] for k in EMBEDDING_KEYS}
    idx = sorted({int(m.group(1)) for k in sd for m in [re.match(r"encoder\.layer\.(\d+)\.", k)] if m})
    if not idx or idx != list(range(len(idx))):
        raise KeyError("encoder.layer.N.* keys are missing or not consecutive: %s" % idx)
    layers = []
    for i in idx:
        p = {}
        for k in _LAYER_KEYS:
            full = "encoder.layer.%d.%s" % (i, k)
            if full not in sd:
                raise KeyError("checkpoint lacks %s" % full)
            p[k] = sd[full]
        t = lambda w: torch.t(w).contiguous()                 # nn.Linear keeps [out, in]
        layers.append({
            "qkv_weight": t(torch.cat((p["attention.self.query.weight"], p["attention.self.key.weight"],
                                       p["attention.self.value.weight"]), 0)),
            "qkv_bias": torch.cat((p["attention.self.query.bias"], p["attention.self.key.bias"],
                                   p["attention.self.value.bias"]), 0),
            "attn_out_weight": t(p["attention.output.dense.weight"]), "attn_out_bias": p["attention.output.dense.bias"],
            "attn_ln_weight": p["attention.output.LayerNorm.weight"], "attn_ln_bias": p["attention.output.LayerNorm.bias"],
            "inter_weight": t(p["intermediate.dense.weight"]), "inter_bias": p["intermediate.dense.bias"],
            "out_weight": t(p["output.dense.weight"]), "out_bias": p["output.dense.bias"],
            "out_ln_weight": p["output.LayerNorm.weight"], "out_ln_bias": p["output.LayerNorm.bias"],
        })
    hidden = emb["word_embeddings.weight"].shape[1]
    for i, w in enumerate(layers):
        if w["qkv_weight"].shape != (hidden, 3 * hidden) or w["out_weight"].shape[1] != hidden:
            raise ValueError("layer %d has shapes that do not fit hidden=%d" % (i, hidden))
    return emb, layers


def pooler_from_state_dict(sd):
    """-> (weight [in, out], bias) of the pooling head, or None when the checkpoint has none.
    BigBird keeps it as `pooler.weight` (an nn.Linear), BERT as `pooler.dense.weight`."""
    sd = _strip_prefix(sd)
    for stem in ("pooler.", "pooler.dense."):
        if stem + "weight" in sd and stem + "bias" in sd:
            return torch.t(sd[stem + "weight"]).contiguous(), sd[stem + "bias"]
    return None


def load(path):
    """-> (embeddings, layers, config) of a local checkpoint; see convert_state_dict."""
    sd, cfg = read_state_dict(path)
    emb, layers = convert_state_dict(sd)
    return emb, layers, cfg
