"""The streaming GPU converter and the direct HF loader against the host converter, and the optional Q4_0 vocabulary
projection.  The checkpoints are small synthetic ones written in the HF layout (key names of LlamaForCausalLM, .bin and
.safetensors shards): the real weights are not available offline."""
import os

import pytest
import torch

from oracle import q40_oracle as O

pytestmark = pytest.mark.gpu

CFG = dict(dim=256, n_layers=2, n_heads=2, vocab_size=320, multiple_of=128, max_batch_size=3, max_seq_len=8, max_prompt_seq_len=16)


def _hf_checkpoint(tmp_path, dtype, fmt, seed=0):
    """two shards with HF key names; returns the directory"""
    g = torch.Generator().manual_seed(seed)
    ffn = O.ffn_hidden_dim(CFG["dim"], CFG["multiple_of"], None)
    d = CFG["dim"]
    sd = {"model.embed_tokens.weight": (torch.randn((CFG["vocab_size"], d), generator=g) * 0.02).to(dtype),
          "lm_head.weight": (torch.randn((CFG["vocab_size"], d), generator=g) * 0.02).to(dtype),
          "model.norm.weight": torch.ones(d, dtype=dtype)}
    for i in range(CFG["n_layers"]):
        p = f"model.layers.{i}."
        sd[p + "input_layernorm.weight"] = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype)
        sd[p + "post_attention_layernorm.weight"] = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype)
        for name, shape in (("self_attn.q_proj", (d, d)), ("self_attn.k_proj", (d, d)), ("self_attn.v_proj", (d, d)), ("self_attn.o_proj", (d, d)),
                            ("mlp.gate_proj", (ffn, d)), ("mlp.down_proj", (d, ffn)), ("mlp.up_proj", (ffn, d))):
            sd[p + name + ".weight"] = (torch.randn(shape, generator=g) * 0.05).to(dtype)
    keys = list(sd)
    shards = [dict((k, sd[k]) for k in keys[: len(keys) // 2]), dict((k, sd[k]) for k in keys[len(keys) // 2:])]
    out = tmp_path / f"hf_{fmt}_{str(dtype)[6:]}"
    os.makedirs(out)
    for n, shard in enumerate(shards):
        if fmt == "bin":
            torch.save(shard, out / f"pytorch_model-{n + 1:05d}-of-00002.bin")
        else:
            from safetensors.torch import save_file
            save_file({k: v.contiguous() for k, v in shard.items()}, str(out / f"model-{n + 1:05d}-of-00002.safetensors"))
    return str(out)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("fmt", ["bin", "safetensors"])
def test_streaming_converter_equals_host_converter(tmp_path, dtype, fmt):
    from spec_mcts_amd import fp16_to_int4 as C
    d = _hf_checkpoint(tmp_path, dtype, fmt)
    got = C.convert_checkpoint_streaming(d, str(tmp_path / "q40.pth"))
    # the host converter on the same tensors (it walks .bin shards only, so feed it the tensors directly)
    want = {}
    for name, v in C.iter_checkpoint_tensors(d):
        want.update(C.quantize_state_dict({name: v}))
    assert sorted(got) == sorted(want) and len(got) == 3 + CFG["n_layers"] * (2 + 7 * 3)
    for k in want:
        if k.endswith(".shape"):
            assert tuple(got[k]) == tuple(want[k])
        else:
            assert got[k].dtype == want[k].dtype and torch.equal(got[k].view(torch.uint8) if got[k].dtype != torch.int8 else got[k],
                                                                 want[k].view(torch.uint8) if want[k].dtype != torch.int8 else want[k]), k
    # and against the oracle's quantiser for one weight
    name = "layers.1.feed_forward.w2"
    v = dict(C.iter_checkpoint_tensors(d))[name + ".weight"]
    w, s, shp = O.quantize_weight(v)
    assert torch.equal(got[name + ".w"], w) and torch.equal(got[name + ".s"].view(torch.int16), s.view(torch.int16)) and tuple(got[name + ".shape"]) == tuple(shp)
    saved = torch.load(str(tmp_path / "q40.pth"), weights_only=True)
    assert torch.equal(saved[name + ".w"], w)


def test_direct_hf_loader_equals_convert_then_load(tmp_path):
    from spec_mcts_amd import ModelArgs, fp16_to_int4 as C
    from spec_mcts_amd.load_q40 import load_hf_q40, load_q40
    d = _hf_checkpoint(tmp_path, torch.bfloat16, "bin", seed=3)
    a = load_hf_q40(d, ModelArgs(**CFG))
    b = load_q40(C.convert_checkpoint_streaming(d), ModelArgs(**CFG))
    prompt = torch.randint(0, CFG["vocab_size"], (1, 11), generator=torch.Generator().manual_seed(4)).cuda()
    la, lb = a(prompt, 0), b(prompt, 0)
    assert torch.equal(la, lb)
    tok = torch.randint(0, CFG["vocab_size"], (3, 1), generator=torch.Generator().manual_seed(5)).cuda()
    assert torch.equal(a(tok, 11), b(tok, 11))
    # ... and the oracle on the converted state dict
    sd = C.convert_checkpoint_streaming(d)
    sd = {k: (v.to(torch.float16) if torch.is_tensor(v) and v.is_floating_point() else v) for k, v in sd.items()}
    oracle = O.OracleTransformer(O.OracleArgs(**CFG), sd, dense=True)
    want = oracle.forward(prompt.cpu(), 0)
    assert torch.allclose(la.cpu().float(), want.float(), rtol=2e-2, atol=2e-2)


def test_q40_lm_head_option():
    from spec_mcts_amd import ModelArgs
    from spec_mcts_amd.load_q40 import load_q40
    cfg = dict(CFG, vocab_size=32016, n_layers=1)
    sd = O.random_q40_state_dict(O.OracleArgs(**cfg), seed=9, std=0.05)
    model = load_q40(dict(sd), ModelArgs(**cfg))
    prompt = torch.randint(0, 32016, (1, 7), generator=torch.Generator().manual_seed(10)).cuda()
    ref = model(prompt, 0)
    model.quantize_lm_head()
    assert model._q40_output[2] == 32128
    model.resetSeq()
    got = model(prompt, 0)
    assert got.shape == ref.shape == (1, 7, 32016)
    # the same hidden state through the dequantised padded weight, in double precision
    w, s, padded = model._q40_output
    deq = O.dequantize_q40(w.cpu(), s.cpu(), 64, (cfg["dim"], padded)).double()
    assert float(deq[:, 32016:].abs().max()) == 0.0
    # the two heads differ by the weight's 4-bit quantisation error: ~0.15 of a weight's standard deviation per weight, so
    # ~0.12 of the logits' standard deviation per logit (sanity bound; the exact check of the projection follows)
    diff = (got.float() - ref.float()).abs()
    assert float(diff.mean()) < 0.2 * float(ref.float().std()) and float(diff.max()) < float(ref.float().std())
    # the projection itself against the oracle's Q4_0 matmul on the padded weight (1e-2 relative / 2e-3 absolute)
    x = torch.randn((5, cfg["dim"]), generator=torch.Generator().manual_seed(12)).half()
    want = O.matmul_q40(x, w.cpu(), s.cpu(), (cfg["dim"], padded))[:, :32016].float()
    head = model._lm_head(x.cuda()).cpu().float()
    assert head.shape == (5, 32016) and bool(((head - want).abs() <= 2e-3 + 1e-2 * want.abs()).all())
    tok = torch.randint(0, 32016, (3, 1), generator=torch.Generator().manual_seed(11)).cuda()
    assert model(tok, 7).shape == (3, 1, 32016)
    model.quantize_lm_head(False)
    model.resetSeq()
    assert torch.equal(model(prompt, 0), ref)
