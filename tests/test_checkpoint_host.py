"""Host logic of the local checkpoint reader: key mapping and re-layout (no GPU, no extension)."""
import importlib.util
import json
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("rt_checkpoint", os.path.join(ROOT, "raptor-t_amd", "checkpoint.py"))
ck = importlib.util.module_from_spec(spec)
spec.loader.exec_module(ck)


def hf_state_dict(hidden=16, ffn=24, layers=2, prefix="", seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)
    sd = {prefix + "embeddings.word_embeddings.weight": r(11, hidden),
          prefix + "embeddings.position_embeddings.weight": r(7, hidden),
          prefix + "embeddings.token_type_embeddings.weight": r(2, hidden),
          prefix + "embeddings.LayerNorm.weight": r(hidden), prefix + "embeddings.LayerNorm.bias": r(hidden)}
    for i in range(layers):
        b = prefix + "encoder.layer.%d." % i
        for name in ("attention.self.query", "attention.self.key", "attention.self.value", "attention.output.dense"):
            sd[b + name + ".weight"], sd[b + name + ".bias"] = r(hidden, hidden), r(hidden)
        sd[b + "intermediate.dense.weight"], sd[b + "intermediate.dense.bias"] = r(ffn, hidden), r(ffn)
        sd[b + "output.dense.weight"], sd[b + "output.dense.bias"] = r(hidden, ffn), r(hidden)
        for ln in ("attention.output.LayerNorm", "output.LayerNorm"):
            sd[b + ln + ".weight"], sd[b + ln + ".bias"] = r(hidden), r(hidden)
    sd[prefix + "pooler.weight"] = r(hidden, hidden)           # ignored by convert_state_dict
    return sd


def test_pooler_head_is_found_in_both_spellings():
    sd = hf_state_dict(prefix="bert.")
    assert ck.pooler_from_state_dict(sd) is None               # a weight without its bias is not a head
    sd["bert.pooler.bias"] = torch.arange(16.0)
    w, b = ck.pooler_from_state_dict(sd)
    x = torch.randn(3, 16)
    assert torch.allclose(x @ w + b, torch.nn.functional.linear(x, sd["bert.pooler.weight"], sd["bert.pooler.bias"]))
    bert = {k.replace("pooler.", "pooler.dense."): v for k, v in sd.items()}
    w2, b2 = ck.pooler_from_state_dict(bert)
    assert torch.equal(w, w2) and torch.equal(b, b2)


@pytest.mark.parametrize("prefix", ["", "bert."])
def test_mapping_reproduces_linear_layers(prefix):
    """x @ converted_weight + bias must equal what nn.Linear computes with the checkpoint's [out, in] weight:
    a missing transpose or a Q/K/V order mix-up fails this."""
    sd = hf_state_dict(prefix=prefix)
    emb, layers = ck.convert_state_dict(sd)
    assert len(layers) == 2 and set(emb) == set(ck.EMBEDDING_KEYS)
    x = torch.randn(5, 16, generator=torch.Generator().manual_seed(9))
    lin = torch.nn.functional.linear
    for i, w in enumerate(layers):
        b = prefix + "encoder.layer.%d." % i
        q, k, v = (x @ w["qkv_weight"] + w["qkv_bias"]).split(16, dim=1)
        for got, name in ((q, "query"), (k, "key"), (v, "value")):
            want = lin(x, sd[b + "attention.self.%s.weight" % name], sd[b + "attention.self.%s.bias" % name])
            assert torch.allclose(got, want, atol=1e-5)
        h = x @ w["inter_weight"] + w["inter_bias"]
        assert torch.allclose(h, lin(x, sd[b + "intermediate.dense.weight"], sd[b + "intermediate.dense.bias"]), atol=1e-5)
        assert torch.allclose(h @ w["out_weight"] + w["out_bias"],
                              lin(h, sd[b + "output.dense.weight"], sd[b + "output.dense.bias"]), atol=1e-5)
        assert torch.equal(w["attn_ln_weight"], sd[b + "attention.output.LayerNorm.weight"])
        assert torch.equal(w["out_ln_bias"], sd[b + "output.LayerNorm.bias"])
    assert torch.equal(emb["position_embeddings.weight"], sd[prefix + "embeddings.position_embeddings.weight"])


def test_reads_safetensors_and_bin_directories(tmp_path):
    from safetensors.torch import save_file
    sd = hf_state_dict(seed=3)
    d1 = tmp_path / "st"
    d1.mkdir()
    save_file({k: v.contiguous() for k, v in sd.items()}, str(d1 / "model.safetensors"))
    (d1 / "config.json").write_text(json.dumps({"num_attention_heads": 2, "layer_norm_eps": 1e-12}))
    emb, layers, cfg = ck.load(str(d1))
    assert cfg["num_attention_heads"] == 2 and len(layers) == 2
    d2 = tmp_path / "bin"
    d2.mkdir()
    torch.save(sd, str(d2 / "pytorch_model.bin"))
    emb2, layers2, cfg2 = ck.load(str(d2))
    assert cfg2 == {} and torch.equal(layers[1]["qkv_weight"], layers2[1]["qkv_weight"])
    assert torch.equal(emb["word_embeddings.weight"], emb2["word_embeddings.weight"])
    emb3, _, _ = ck.load(str(d1 / "model.safetensors"))
    assert torch.equal(emb3["LayerNorm.bias"], emb["LayerNorm.bias"])


def test_errors_name_what_is_missing(tmp_path):
    sd = hf_state_dict()
    del sd["encoder.layer.1.output.dense.bias"]
    with pytest.raises(KeyError, match="encoder.layer.1.output.dense.bias"):
        ck.convert_state_dict(sd)
    with pytest.raises(KeyError, match="word_embeddings"):
        ck.convert_state_dict({"foo": torch.zeros(1)})
    gap = {k.replace("layer.1.", "layer.3."): v for k, v in hf_state_dict().items()}
    with pytest.raises(KeyError, match="consecutive"):
        ck.convert_state_dict(gap)
    with pytest.raises(FileNotFoundError):
        ck.load(str(tmp_path))
