"""Host side of the checkpoint path: shard iteration (memory-mapped .bin and safetensors), HF -> Meta key names, the
host converter's output format (fp16_to_int4.py:165-184: <name>.w / .s / .shape, everything else as loaded)."""
import os

import torch

from oracle import q40_oracle as O


def _write(tmp_path, fmt):
    g = torch.Generator().manual_seed(1)
    sd = {"model.embed_tokens.weight": torch.randn((40, 128), generator=g).to(torch.bfloat16),
          "model.layers.0.self_attn.q_proj.weight": (torch.randn((128, 128), generator=g) * 0.05).to(torch.bfloat16),
          "model.layers.0.mlp.down_proj.weight": (torch.randn((128, 256), generator=g) * 0.05).to(torch.bfloat16),
          "model.layers.0.input_layernorm.weight": torch.ones(128, dtype=torch.bfloat16),
          "lm_head.weight": torch.randn((40, 128), generator=g).to(torch.bfloat16)}
    d = tmp_path / fmt
    os.makedirs(d)
    if fmt == "bin":
        torch.save(sd, d / "pytorch_model-00001-of-00001.bin")
    else:
        from safetensors.torch import save_file
        save_file(sd, str(d / "model-00001-of-00001.safetensors"))
    return str(d), sd


def test_shard_iteration_renames_keys_and_keeps_tensors(tmp_path):
    from spec_mcts_amd import fp16_to_int4 as C
    for fmt in ("bin", "safetensors"):
        d, sd = _write(tmp_path, fmt)
        got = dict(C.iter_checkpoint_tensors(d))
        assert sorted(got) == ["layers.0.attention.wq.weight", "layers.0.attention_norm.weight", "layers.0.feed_forward.w2.weight",
                               "output.weight", "tok_embeddings.weight"]
        assert torch.equal(got["layers.0.feed_forward.w2.weight"], sd["model.layers.0.mlp.down_proj.weight"])
        assert C._is_quantised_key("layers.0.attention.wq.weight") and not C._is_quantised_key("layers.0.attention_norm.weight")
        assert not C._is_quantised_key("output.weight")


def test_host_converter_output_format(tmp_path):
    from spec_mcts_amd import fp16_to_int4 as C
    d, sd = _write(tmp_path, "bin")
    out = C.convert_checkpoint(d, str(tmp_path / "out.pth"))
    assert sorted(out) == ["layers.0.attention.wq.s", "layers.0.attention.wq.shape", "layers.0.attention.wq.w", "layers.0.attention_norm.weight",
                           "layers.0.feed_forward.w2.s", "layers.0.feed_forward.w2.shape", "layers.0.feed_forward.w2.w", "output.weight",
                           "tok_embeddings.weight"]
    v = sd["model.layers.0.mlp.down_proj.weight"]
    w, s, shp = O.quantize_weight(v)                                  # the oracle's restatement of quantize_q40(v.t(), 64)
    assert torch.equal(out["layers.0.feed_forward.w2.w"], w) and torch.equal(out["layers.0.feed_forward.w2.s"], s)
    assert tuple(out["layers.0.feed_forward.w2.shape"]) == (128, 256) == tuple(shp)
    assert out["layers.0.feed_forward.w2.w"].shape == (256 * 128 // 128, 64) and out["layers.0.feed_forward.w2.s"].shape == (256 * 128 // 64, 1)
    assert torch.equal(out["output.weight"], sd["lm_head.weight"])
    saved = torch.load(str(tmp_path / "out.pth"), weights_only=True)
    assert torch.equal(saved["layers.0.attention.wq.w"], out["layers.0.attention.wq.w"])
