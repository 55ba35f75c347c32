"""The C-ABI library loads and exports every symbol include/smh.h declares (no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "smh.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(smh_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from spec_mcts_amd import _lib
    names = _declared()
    assert len(names) >= 15
    lib = _lib.load()
    for n in names:
        assert hasattr(lib, n), f"{n} declared in smh.h but not exported by libsmh.so"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature in spec_mcts_amd/_lib.py"
    assert sorted(_lib.SIGNATURES) == names
    assert lib.smh_version() == 1


def test_argument_errors_are_reported_without_a_gpu():
    from spec_mcts_amd import _lib
    lib = _lib.load()
    # N not a multiple of 128 is rejected before anything touches the device
    st = lib.smh_q40_gemv(None, 1, 64, 64, None, None, 100, None, 100, 0, None, 0, None, 0, None)
    assert st < 0 and b"multiple of 128" in lib.smh_last_error_string()
    st = lib.smh_q40_quantize(None, None, None, 3, None)
    assert st < 0 and b"even" in lib.smh_last_error_string()
    with pytest.raises(_lib.SmhError):
        _lib.check(st, "smh_q40_quantize")
    assert lib.smh_q40_matmul_workspace_bytes(16, 4096) >= 16 * 16 * 4096 * 4
    import ctypes
    n = (ctypes.c_int * 3)(4096, 4096, 4096)
    ks = lib.smh_q40_matmul_plan(1, 4096, 3, n)
    assert 1 <= ks <= 16
    assert lib.smh_q40_matmul_plan(1, 4096, 1, (ctypes.c_int * 1)(100)) < 0      # N not a multiple of 128
    assert lib.smh_attn_workspace_bytes(64, 32, 1024) >= 32 * 64 * 32 * 130 * 4
    # SwiGLU inside the gate|up launch: 17 .. 128 rows, K a multiple of 64, at most 16384 columns per weight
    assert lib.smh_q40_swiglu_fits(100, 4096, 11008) == 1 and lib.smh_q40_swiglu_fits(16, 4096, 11008) == 0
    assert lib.smh_q40_swiglu_fits(100, 4096, 28672) == 0 and lib.smh_q40_swiglu_fits(100, 4096, 1024) == 0
    st = lib.smh_q40_matmul_tiled_swiglu(None, 5, 4096, 4096, None, None, 11008, None, 11008, None)
    assert st < 0 and b"17 .. 128" in lib.smh_last_error_string()
    # the entry point without a workspace refuses shapes beyond its static array before anything touches the device
    assert lib.smh_attn_static_scratch_bytes() == 16 << 20
    st = lib.smh_shared_prefix_attn_static(None, None, 4096, 64, 64, 128, None, None, 4096, 0, None, None, None, None, 0, None, 0,
                                           None, None, None)
    assert st < 0 and b"static array holds" in lib.smh_last_error_string()


def test_matmul_plans_fit_the_workspace_the_library_asks_for():
    """the slabs of any planned launch (even split, or runs of steps across column units above 16 rows) fit the bytes
    smh_q40_matmul_workspace_bytes returns for the largest batch and width, and never exceed 16 slices"""
    from spec_mcts_amd import _lib
    lib = _lib.load()
    widths = ([4096], [4096, 4096, 4096], [11008, 11008], [11008], [32128], [8192, 1024, 1024], [28672, 28672], [16640, 16640],
              [7680, 7680, 7680], [128], [256, 128, 128])
    for K in (32, 256, 1024, 2048, 4096, 8192, 11008, 28672):
        for ns in widths:
            n = (ctypes.c_int * len(ns))(*ns)
            for M in (1, 2, 10, 16, 17, 64, 100, 128):
                for plan in (lib.smh_q40_matmul_plan, lib.smh_q40_matmul_plan_tiled):
                    ks = plan(M, K, len(ns), n)
                    assert 1 <= ks <= 16, (M, K, ns, ks)
                    assert ks * M * sum(ns) * 4 <= lib.smh_q40_matmul_workspace_bytes(M, sum(ns)), (M, K, ns, ks)
                if M <= 16:
                    assert lib.smh_q40_matmul_plan(M, K, len(ns), n) == lib.smh_q40_matmul_plan_tiled(M, K, len(ns), n)
    # the plans the GPU tests and the design notes name: checkpoint layout ...
    three, two, one = (ctypes.c_int * 3)(4096, 4096, 4096), (ctypes.c_int * 2)(11008, 11008), (ctypes.c_int * 1)(4096)
    assert lib.smh_q40_matmul_plan(100, 4096, 2, two) == 4      # range cut: 256 runs of 43 steps
    assert lib.smh_q40_matmul_plan(100, 4096, 3, three) == 5
    # ... and tiled weights at 100 rows: 128-column blocks with two K-groups a workgroup
    assert lib.smh_q40_matmul_plan_tiled(100, 4096, 1, one) == 4         # wo: 32 blocks x 2 row blocks x 4 slices
    assert lib.smh_q40_matmul_plan_tiled(100, 11008, 1, one) == 8        # w2: 32 blocks x 8 slices
    assert lib.smh_q40_matmul_plan_tiled(100, 4096, 3, three) == 2       # wq|wk|wv: 96 blocks x 2 slices
    assert lib.smh_q40_matmul_plan_tiled(100, 4096, 2, two) == 1         # w1|w3: 172 blocks, K uncut
    assert lib.smh_q40_matmul_plan_tiled(32, 4096, 2, two) == 4          # wide and at most 64 rows: the 256-column units' plan


def test_host_quantiser_matches_oracle():
    """spec_mcts_amd.quant (the converter's quantiser) against the oracle on the host"""
    import torch
    from oracle import q40_oracle as O
    from spec_mcts_amd import quant
    g = torch.Generator().manual_seed(5)
    v = (torch.randn((256, 128), generator=g) * 0.02).to(torch.float16)
    w, s, shp = quant.quantize_linear_weight(v)
    w2, s2, shp2 = O.quantize_weight(v)
    assert torch.equal(w, w2) and torch.equal(s, s2) and shp == shp2
    assert torch.equal(quant.dequantize_q40_torch(w, s, 64, (128, 256)), O.dequantize_q40(w, s, 64, (128, 256)))
    vb = v.to(torch.bfloat16)
    wb, sb = quant.quantize_q40_torch(vb.t(), 64)
    wb2, sb2 = O.quantize_q40(vb.t(), 64)
    assert torch.equal(wb, wb2) and torch.equal(sb, sb2)


def test_converter_and_loader_host_logic():
    import torch
    from spec_mcts_amd import fp16_to_int4 as C
    from spec_mcts_amd.load_q40 import load_q40
    from spec_mcts_amd import ModelArgs
    g = torch.Generator().manual_seed(6)
    hf = {"model.embed_tokens.weight": torch.randn((320, 256), generator=g).half(),
          "model.norm.weight": torch.ones(256).half(), "lm_head.weight": torch.randn((320, 256), generator=g).half()}
    for name, shape in (("self_attn.q_proj", (256, 256)), ("self_attn.k_proj", (256, 256)), ("self_attn.v_proj", (256, 256)),
                        ("self_attn.o_proj", (256, 256)), ("mlp.gate_proj", (768, 256)), ("mlp.down_proj", (256, 768)),
                        ("mlp.up_proj", (768, 256))):
        hf[f"model.layers.0.{name}.weight"] = (torch.randn(shape, generator=g) * 0.02).half()
    hf["model.layers.0.input_layernorm.weight"] = torch.ones(256).half()
    hf["model.layers.0.post_attention_layernorm.weight"] = torch.ones(256).half()
    sd = C.quantize_state_dict(C.remap_state_dict(hf))
    assert "layers.0.attention.wq.w" in sd and "layers.0.feed_forward.w2.shape" in sd and "tok_embeddings.weight" in sd
    assert "layers.0.attention.wq.weight" not in sd and tuple(sd["layers.0.feed_forward.w1.shape"]) == (768, 256)
    args = ModelArgs(dim=256, n_layers=1, n_heads=2, vocab_size=320, multiple_of=128, max_batch_size=2, max_seq_len=4,
                     max_prompt_seq_len=8)
    model = load_q40(sd, args, device="cpu")
    lin = model.layers[0].feed_forward.w2
    assert tuple(lin.shape) == (256, 768) and lin.w.shape == (768 * 256 // 128, 64) and lin.s.numel() == 768 * 256 // 64
    assert model.tok_embeddings.weight.dtype == torch.float16 and model.output.weight.shape == (320, 256)
    # the hot path refuses to run without a GPU instead of falling back
    with pytest.raises(AssertionError):
        model(torch.zeros((1, 4), dtype=torch.int64), 0)
