"""On-disk format and model surgery (host logic; CPU)."""
import json
import os

import pytest
import torch
import torch.nn as nn

import utils as cq_utils
from llama.cherry_linear import QuantLinear as TrainLinear
from llama.qlinear import QuantLinear


class Block(nn.Module):
    def __init__(self, bits):
        super().__init__()
        kw = dict(bias=False, w_bits=bits, group_size=128, cherryq=True, cherry_fraction=1 / 32)
        self.q_proj = TrainLinear(256, 256, **kw)
        self.inner = nn.Sequential(TrainLinear(256, 512, **kw), nn.SiLU(), TrainLinear(512, 256, **kw))
        self.plain = nn.Linear(256, 8)


def _register(model, seed=0):
    g = torch.Generator().manual_seed(seed)
    for m in model.modules():
        if isinstance(m, TrainLinear):
            with torch.no_grad():
                m.weight.copy_(torch.randn(m.weight.shape, generator=g) * 0.02)
            m.register_cherry_indices(torch.randperm(m.in_features, generator=g)[:m.num_cherries])


@pytest.mark.parametrize("bits", [3, 4])
def test_make_quant_and_pack_model(bits):
    model = Block(bits).half()
    _register(model)
    dense = {n: m._adjust_weight(m.weight, ste=False).detach().clone()
             for n, m in model.named_modules() if isinstance(m, TrainLinear)}
    assert set(dense) == {"q_proj", "inner.0", "inner.2"}
    cq_utils.pack_model(model)
    packed = {n: m for n, m in model.named_modules() if isinstance(m, QuantLinear)}
    assert set(packed) == set(dense)
    assert isinstance(model.plain, nn.Linear) and not any(isinstance(m, TrainLinear) for m in model.modules())
    for n, m in packed.items():
        assert m.qweight.shape == ((m.in_features - m.num_cherries) // 8 * bits, m.out_features)
        assert m.qweight.dtype == torch.uint8 and m.cherry_indices.dtype == torch.int16
        assert m.bias is None
        w = m.unpack()
        # equal except at rounding ties of the quantiser (one grid step, < 0.5 % of entries)
        diff = (w.float() - dense[n].float()).abs()
        assert (diff > 0).float().mean() < 5e-3
    keys = set(model.state_dict())
    for n in packed:
        for b in ("cherry_indices", "cherry_weight", "qweight", "scales"):
            assert f"{n}.{b}" in keys


def test_save_and_load_decoder_roundtrip(tmp_path):
    import cherryq_decoder as cd
    cfg = cd.DecoderConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=2,
                           num_key_value_heads=2, vocab_size=128, max_position_embeddings=16, w_bits=3,
                           group_size=128, cherry_fraction=1 / 16)
    model = cd.CherryLlamaDecoder(cfg, seed=1, device="cpu")
    path = cq_utils.save_quantized(model, str(tmp_path))
    assert os.path.basename(path) == "pytorch_model-3bit-128g.bin"
    conf = json.load(open(tmp_path / "config.json"))
    assert conf["w_bits"] == 3 and conf["group_size"] == 128 and conf["hidden_size"] == 256
    sd = torch.load(path, weights_only=True)
    assert "model.layers.1.self_attn.k_proj.qweight" in sd and "model.layers.0.mlp.down_proj.scales" in sd
    assert "model.embed_tokens.weight" in sd and "lm_head.weight" in sd and "model.norm.weight" in sd
    assert sd["model.layers.0.mlp.gate_proj.cherry_indices"].dtype == torch.int16
    loaded = cq_utils.from_quantized(str(tmp_path), device_map="cpu")
    a, b = model.reference_state_dict(), loaded.reference_state_dict()
    assert a.keys() == b.keys()
    for k in a:
        assert torch.equal(a[k], b[k]), k
    # a checkpoint from an older transformers version also carries rotary buffers: ignored
    sd["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(64)
    loaded.load_reference_state_dict(sd)
    sd["bogus"] = torch.zeros(1)
    with pytest.raises(KeyError):
        loaded.load_reference_state_dict(sd)
    del sd["bogus"]
    sd["model.norm.weight"] = torch.zeros(3, dtype=torch.float16)
    with pytest.raises(ValueError):
        loaded.load_reference_state_dict(sd)
