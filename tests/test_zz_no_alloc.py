"""smh_shared_prefix_attn_static (the entry point that allocates nothing: its prefix partials live in a static device
array of the library) against smh_shared_prefix_attn (caller's workspace): same kernels, same plan, so the outputs
must be bit-identical - on two calls in a row, the second with a smaller input that leaves stale partials of the first
call in the array."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(B, H, Hkv, P, S, seed, q40):
    g = torch.Generator().manual_seed(seed)
    dev = "cuda:0"
    q = torch.randn((B, H, 128), generator=g).half().to(dev)
    pk = torch.randn((max(P, 1), Hkv, 128), generator=g).half().to(dev)
    pv = torch.randn((max(P, 1), Hkv, 128), generator=g).half().to(dev)
    lens = torch.randint(0, S + 1, (B,), generator=g, dtype=torch.int32).to(dev)
    ck = torch.randn((B, Hkv, 128), generator=g).half().to(dev)
    cv = torch.randn((B, Hkv, 128), generator=g).half().to(dev)
    if q40:
        sk = torch.randint(-128, 128, (B, S, Hkv, 64), generator=g, dtype=torch.int16).to(torch.int8).to(dev)
        sv = torch.randint(-128, 128, (B, S, Hkv, 64), generator=g, dtype=torch.int16).to(torch.int8).to(dev)
        sks = (torch.rand((B, S, Hkv, 2), generator=g) * 0.2).half().to(dev)
        svs = (torch.rand((B, S, Hkv, 2), generator=g) * 0.2).half().to(dev)
    else:
        sk = torch.randn((B, S, Hkv, 128), generator=g).half().to(dev)
        sv = torch.randn((B, S, Hkv, 128), generator=g).half().to(dev)
        sks = svs = None
    return dict(q=q, prefix_k=pk, prefix_v=pv, P=P, suffix_k=sk, suffix_v=sv, suffix_ks=sks, suffix_vs=svs, Smax=S, lens=lens,
                lens_stride=1, cur_k=ck, cur_v=cv)


def test_static_scratch_entry_point_matches_workspace_entry_point():
    from spec_mcts_amd import _lib, kernels as K
    lib = _lib.load()
    assert lib.smh_attn_static_scratch_bytes() == 16 << 20
    # the first call is the larger one (64 branches x 32 heads, 1024-token prefix, Q4_0 suffixes: 8.5 MB of partials);
    # the second is smaller in every dimension (grouped-query heads, fp16 suffixes) and runs over the first call's leftovers
    cases = [_case(64, 32, 32, 1024, 96, 11, True), _case(5, 16, 4, 300, 17, 12, False)]
    for rnd in range(2):
        for kw in cases:
            args = dict(kw)
            q = args.pop("q")
            want = K.shared_prefix_attn(q, args.pop("prefix_k"), args.pop("prefix_v"), args.pop("P"), **args)
            args = dict(kw)
            q = args.pop("q")
            out = torch.full_like(q, float("nan"))
            torch.cuda.synchronize()
            before = torch.cuda.memory_stats()["allocation.all.allocated"]      # allocation events so far
            got = K.shared_prefix_attn(q, args.pop("prefix_k"), args.pop("prefix_v"), args.pop("P"), out=out, static_scratch=True, **args)
            assert torch.cuda.memory_stats()["allocation.all.allocated"] == before, "the static entry point's wrapper must not allocate"
            torch.cuda.synchronize()
            assert got.data_ptr() == out.data_ptr()
            assert torch.isfinite(got.float()).all()
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"round {rnd}: outputs differ"


def test_static_scratch_entry_point_rejects_shapes_beyond_its_array():
    from spec_mcts_amd import _lib, kernels as K
    kw = _case(2, 2, 2, 64, 4, 13, False)
    lib = _lib.load()
    # 4096 branches x 64 heads over a 4096-token prefix would need 4 GB of partials
    st = lib.smh_shared_prefix_attn_static(kw["q"].data_ptr(), kw["q"].data_ptr(), 4096, 64, 64, 128, kw["prefix_k"].data_ptr(),
                                           kw["prefix_v"].data_ptr(), 4096, 0, None, None, None, None, 0, None, 0, None, None, None)
    assert st < 0 and b"static array holds" in lib.smh_last_error_string()
