"""GPU parity of the shared-prefix decode attention and the causal prefill attention against the
oracle (explicit fp32 softmax attention).  Tolerance: 1e-2 relative + 2e-3 absolute."""
import pytest
import torch

from oracle import q40_oracle as O

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 2e-3


def _g(seed):
    return torch.Generator().manual_seed(seed)


def _check(got, want):
    got, want = got.float().cpu(), want.float()
    err = (got - want).abs()
    tol = ATOL + RTOL * want.abs()
    assert bool((err <= tol).all()), f"max err {err.max():.4e}, worst excess {(err - tol).max():.4e}"


def _inputs(B, H, Hkv, D, P, S, seed, std=1.0):
    g = _g(seed)
    q = (torch.randn((B, H, D), generator=g) * std).to(torch.float16)
    pk = (torch.randn((max(P, 1), Hkv, D), generator=g) * std).to(torch.float16)
    pv = (torch.randn((max(P, 1), Hkv, D), generator=g) * std).to(torch.float16)
    sk = (torch.randn((B, max(S, 1), Hkv, D), generator=g) * std).to(torch.float16)
    sv = (torch.randn((B, max(S, 1), Hkv, D), generator=g) * std).to(torch.float16)
    lens = torch.randint(0, S + 1, (B,), generator=g, dtype=torch.int32)
    return q, pk, pv, sk, sv, lens


def test_config2_fp16_suffix():
    """B=64 branches, 32 heads, D=128, shared 1024-token prefix, ragged suffix 0..256, seed 2"""
    from spec_mcts_amd import kernels as K
    B, H, D, P, S = 64, 32, 128, 1024, 256
    q, pk, pv, sk, sv, lens = _inputs(B, H, H, D, P, S, 2)
    lens[0] = 0; lens[1] = S
    got = K.shared_prefix_attn(q.cuda(), pk.cuda(), pv.cuda(), P, suffix_k=sk.cuda(), suffix_v=sv.cuda(),
                               Smax=S, lens=lens.cuda(), lens_stride=1)
    want = O.shared_prefix_attention(q, pk, pv, sk, sv, lens.tolist())
    _check(got, want)


def test_config2_q40_suffix_as_the_model_stores_it():
    from spec_mcts_amd import kernels as K
    B, H, D, P, S = 64, 32, 128, 1024, 256
    q, pk, pv, sk, sv, lens = _inputs(B, H, H, D, P, S, 3)
    wk, sks = O.quantize_q40(sk, 64)
    wv, svs = O.quantize_q40(sv, 64)
    sk_deq = O.dequantize_q40(wk, sks, 64, sk.shape)
    sv_deq = O.dequantize_q40(wv, svs, 64, sv.shape)
    got = K.shared_prefix_attn(q.cuda(), pk.cuda(), pv.cuda(), P, suffix_k=wk.cuda(), suffix_v=wv.cuda(),
                               suffix_ks=sks.cuda(), suffix_vs=svs.cuda(), Smax=S, lens=lens.cuda(), lens_stride=1)
    want = O.shared_prefix_attention(q, pk, pv, sk_deq, sv_deq, lens.tolist())
    _check(got, want)


@pytest.mark.parametrize("B,H,Hkv,P,S", [(1, 2, 2, 1, 0), (3, 8, 2, 100, 5), (100, 8, 1, 512, 3), (17, 4, 4, 33, 9),
                                         (5, 2, 2, 0, 7), (2, 64, 8, 2048, 4)])
def test_shapes_gqa_empty_prefix_and_current_token(B, H, Hkv, P, S):
    from spec_mcts_amd import kernels as K
    D = 128
    q, pk, pv, sk, sv, lens = _inputs(B, H, Hkv, D, P, S, 10 + B)
    g = _g(99)
    ck = torch.randn((B, Hkv, D), generator=g).to(torch.float16)
    cv = torch.randn((B, Hkv, D), generator=g).to(torch.float16)
    # the new token is one more exact row after each branch's suffix
    sk2 = torch.cat((sk, torch.zeros_like(sk[:, :1])), 1); sv2 = torch.cat((sv, torch.zeros_like(sv[:, :1])), 1)
    for b in range(B):
        sk2[b, lens[b]] = ck[b]; sv2[b, lens[b]] = cv[b]
    want = O.shared_prefix_attention(q, pk[:P], pv[:P], sk2, sv2, (lens + 1).tolist())
    got = K.shared_prefix_attn(q.cuda(), pk.cuda() if P else None, pv.cuda() if P else None, P,
                               suffix_k=sk.cuda(), suffix_v=sv.cuda(), Smax=max(S, 1), lens=lens.cuda(), lens_stride=1,
                               cur_k=ck.cuda(), cur_v=cv.cuda(), n_kv_heads=Hkv)
    _check(got, want)


def test_uniform_length_from_device_counter():
    """lens_stride 0: every branch uses the same device-side step counter, as the model does"""
    from spec_mcts_amd import kernels as K
    B, H, D, P, S = 6, 4, 128, 64, 8
    q, pk, pv, sk, sv, _ = _inputs(B, H, H, D, P, S, 30)
    t = torch.tensor([5], dtype=torch.int32).cuda()
    got = K.shared_prefix_attn(q.cuda(), pk.cuda(), pv.cuda(), P, suffix_k=sk.cuda(), suffix_v=sv.cuda(), Smax=S,
                               lens=t, lens_stride=0)
    _check(got, O.shared_prefix_attention(q, pk, pv, sk, sv, [5] * B))


def test_special_cases():
    from spec_mcts_amd import kernels as K
    B, H, D, P, S = 4, 2, 128, 96, 8
    q, pk, pv, sk, sv, lens = _inputs(B, H, H, D, P, S, 31)
    lens[:] = S
    # q = 0 -> uniform weights -> mean of all V rows
    got = K.shared_prefix_attn(torch.zeros_like(q).cuda(), pk.cuda(), pv.cuda(), P, suffix_k=sk.cuda(),
                               suffix_v=sv.cuda(), Smax=S, lens=lens.cuda(), lens_stride=1).cpu()
    for b in range(B):
        assert torch.allclose(got[b].float(), torch.cat((pv, sv[b]), 0).float().mean(0), atol=2e-3)
    # one dominant prefix key -> its V row
    pk2 = pk.clone(); pk2[70] = 0; pk2[70, :, 0] = 200.0
    q2 = torch.zeros_like(q); q2[..., 0] = 50.0
    got = K.shared_prefix_attn(q2.cuda(), pk2.cuda(), pv.cuda(), P).cpu()
    assert torch.allclose(got[0].float(), pv[70].float(), atol=2e-3)
    # split invariance: moving the tail of the prefix into every branch's suffix changes nothing
    full = K.shared_prefix_attn(q.cuda(), pk.cuda(), pv.cuda(), P, suffix_k=sk.cuda(), suffix_v=sv.cuda(), Smax=S,
                                lens=lens.cuda(), lens_stride=1).cpu()
    cut = 40
    sk2 = torch.cat((pk[cut:][None].expand(B, -1, -1, -1), sk), 1).contiguous()
    sv2 = torch.cat((pv[cut:][None].expand(B, -1, -1, -1), sv), 1).contiguous()
    l2 = (lens + P - cut).to(torch.int32)
    moved = K.shared_prefix_attn(q.cuda(), pk[:cut].contiguous().cuda(), pv[:cut].contiguous().cuda(), cut,
                                 suffix_k=sk2.cuda(), suffix_v=sv2.cuda(), Smax=S + P - cut, lens=l2.cuda(),
                                 lens_stride=1).cpu()
    assert torch.allclose(full.float(), moved.float(), atol=2e-3, rtol=1e-2)


@pytest.mark.parametrize("S,H,Hkv", [(1, 2, 2), (19, 4, 2), (63, 2, 1), (64, 2, 2), (65, 4, 1), (200, 8, 2), (512, 32, 32), (1100, 8, 1)])
def test_prefill_causal(S, H, Hkv):
    from spec_mcts_amd import kernels as K
    g = _g(40 + S)
    q = torch.randn((S, H, 128), generator=g).to(torch.float16)
    k = torch.randn((S, Hkv, 128), generator=g).to(torch.float16)
    v = torch.randn((S, Hkv, 128), generator=g).to(torch.float16)
    got = K.prefill_attn(q.cuda(), k.cuda(), v.cuda())
    _check(got, O.causal_attention(q, k, v))


def test_prefill_causal_special_cases():
    """what the mathematics fixes: position 0 sees only itself (out = v[0]); equal keys give the running mean of v;
    one key that dominates every score makes every later position return that key's v"""
    from spec_mcts_amd import kernels as K
    S, H = 150, 2
    g = _g(77)
    q = torch.randn((S, H, 128), generator=g).half()
    k = torch.randn((S, H, 128), generator=g).half()
    v = torch.randn((S, H, 128), generator=g).half()
    out = K.prefill_attn(q.cuda(), k.cuda(), v.cuda()).cpu()
    assert torch.equal(out[0], v[0])
    k_same = k[:1].expand(S, H, 128).contiguous()
    out = K.prefill_attn(q.cuda(), k_same.cuda(), v.cuda()).cpu().float()
    mean = v.float().cumsum(0) / torch.arange(1, S + 1).view(S, 1, 1)
    assert torch.allclose(out, mean, atol=2e-3, rtol=1e-2)
    k_dom = (torch.randn((S, H, 128), generator=g) * 0.01).half()
    k_dom[70] = q[100] * 4                       # huge score for every query that resembles q[100]; use q = q[100] everywhere
    q_all = q[100:101].expand(S, H, 128).contiguous()
    out = K.prefill_attn(q_all.cuda(), k_dom.cuda(), v.cuda()).cpu().float()
    assert torch.allclose(out[70:], v[70:71].float().expand(S - 70, H, 128), atol=2e-3, rtol=1e-2)


def test_flash_attn_page_flash_attn_and_chunk_attn_drop_ins():
    """the reference's operator names (triton_kernels.py:621, :764) on top of the decode attention kernel, with
    the shapes of its own checks (triton_kernels_bench.py:294-330: B=100, L=512, H=32, D=128, atol 1e-2)"""
    from spec_mcts_amd import kernels as K
    g = torch.Generator().manual_seed(1)
    B, L, H, D = 100, 512, 32, 128
    q = torch.randn((B, H, D), generator=g).half()
    k = torch.randn((B, H, L, D), generator=g).half()
    v = torch.randn((B, H, L, D), generator=g).half()
    got = K.flash_attn(q.cuda(), k.cuda(), v.cuda(), B, L, H, D).cpu()
    want = torch.nn.functional.scaled_dot_product_attention(q.float()[:, :, None], k.float(), v.float())[:, :, 0]
    assert got.dtype == torch.float16 and torch.allclose(got.float(), want, rtol=1e-2, atol=2e-3)
    # paged: a pool of P pages per head, every branch an arbitrary list of L pages (pages may repeat)
    P, B2, L2 = 300, 27, 130
    kp = torch.randn((H, P, D), generator=g).half()
    vp = torch.randn((H, P, D), generator=g).half()
    pager = torch.randint(0, P, (B2, L2), generator=g).to(torch.int16)
    q2 = torch.randn((B2, H, D), generator=g).half()
    got2 = K.page_flash_attn(pager.cuda(), q2.cuda(), kp.cuda(), vp.cuda(), P, B2, L2, H, D).cpu()
    idx = pager.long()
    kk = kp.float()[:, idx].permute(1, 0, 2, 3)           # [B, H, L, D]
    vv = vp.float()[:, idx].permute(1, 0, 2, 3)
    want2 = torch.nn.functional.scaled_dot_product_attention(q2.float()[:, :, None], kk, vv)[:, :, 0]
    assert torch.allclose(got2.float(), want2, rtol=1e-2, atol=2e-3)
    # chunked: pool rows 0..offset-1 shared by every branch, then the branch's own pages; the shapes of the
    # reference's tree-attention check (triton_kernels_bench.py:479-493: 27 branches, 512 rows, 256 shared)
    for offset, L3 in ((256, 512), (0, 40), (40, 40)):
        pager3 = torch.randint(0, P, (B2, L3), generator=g).to(torch.int16)
        pager3[:, :offset] = torch.arange(offset, dtype=torch.int16)
        got3 = K.chunk_attn(pager3.cuda(), q2.cuda(), kp.cuda(), vp.cuda(), P, B2, L3, H, D, offset).cpu()
        idx3 = pager3.long()
        want3 = torch.nn.functional.scaled_dot_product_attention(
            q2.float()[:, :, None], kp.float()[:, idx3].permute(1, 0, 2, 3), vp.float()[:, idx3].permute(1, 0, 2, 3))[:, :, 0]
        assert got3.dtype == torch.float16 and torch.allclose(got3.float(), want3, rtol=1e-2, atol=2e-3)
        if offset:
            same = K.page_flash_attn(pager3.cuda(), q2.cuda(), kp.cuda(), vp.cuda(), P, B2, L3, H, D).cpu()
            assert torch.allclose(got3.float(), same.float(), rtol=1e-2, atol=2e-3)


@pytest.mark.parametrize("B,H,Hkv,P,t", [(1, 4, 4, 40, 0), (3, 4, 4, 40, 5), (16, 8, 2, 100, 9), (5, 8, 8, 0, 3)])
def test_attention_fed_by_the_qkv_product_matches_the_three_launch_sequence(B, H, Hkv, P, t):
    """smh_shared_prefix_attn_qkv (RoPE + KV append inside the attention kernels) against
    smh_partial_rope_append_kv + smh_shared_prefix_attn on the same slabs: same rounding points, so the
    outputs and the appended cache rows must be bit-identical."""
    from spec_mcts_amd import kernels as K
    dev = "cuda:0"
    D, Smax, dim = 128, 16, 512
    g = torch.Generator(device="cpu").manual_seed(900 + B + t)
    x = (torch.randn((B, dim), generator=g) * 0.5).half().to(dev)
    ws = []
    for n in (H * D, Hkv * D, Hkv * D):
        w = torch.randint(-128, 128, (dim * n // 2,), generator=g, dtype=torch.int16).to(torch.int8).to(dev)
        s = (torch.rand((dim * n // 64,), generator=g) * 0.02 + 0.005).half().to(dev)
        ws.append((w, s, n))
    qkv = K.matmul_q40_partial(x, ws)
    ang = torch.rand((64, 64), generator=g) * 6.28
    cos, sin = torch.cos(ang).half().to(dev), torch.sin(ang).half().to(dev)
    pos_dev = torch.tensor([P + t], dtype=torch.int32, device=dev) % 64
    t_dev = torch.tensor([t], dtype=torch.int32, device=dev)
    pk = (torch.randn((max(P, 1), Hkv, D), generator=g) * 0.5).half().to(dev)
    pv = (torch.randn((max(P, 1), Hkv, D), generator=g) * 0.5).half().to(dev)
    caches = []
    for _ in range(2):
        ck = torch.randint(-128, 128, (B, Smax, Hkv, 64), generator=torch.Generator().manual_seed(7), dtype=torch.int16).to(torch.int8).to(dev)
        cv = torch.randint(-128, 128, (B, Smax, Hkv, 64), generator=torch.Generator().manual_seed(8), dtype=torch.int16).to(torch.int8).to(dev)
        cks = (torch.rand((B, Smax, Hkv, 2), generator=torch.Generator().manual_seed(9)) * 0.1 + 0.01).half().to(dev)
        cvs = (torch.rand((B, Smax, Hkv, 2), generator=torch.Generator().manual_seed(10)) * 0.1 + 0.01).half().to(dev)
        caches.append((ck, cks, cv, cvs))
    ck, cks, cv, cvs = caches[0]
    q, k, v = K.partial_rope_append_kv(qkv, H, Hkv, D, cos, sin, pos_dev, ck, cks, cv, cvs, Smax, t_dev)
    want = K.shared_prefix_attn(q, pk if P else None, pv if P else None, P, suffix_k=ck, suffix_v=cv, suffix_ks=cks, suffix_vs=cvs,
                                Smax=Smax, lens=t_dev, lens_stride=0, cur_k=k, cur_v=v, n_kv_heads=Hkv)
    ck2, cks2, cv2, cvs2 = caches[1]
    got = K.shared_prefix_attn_qkv(qkv, H, Hkv, D, cos, sin, pos_dev, pk if P else None, pv if P else None, P,
                                   ck2, cks2, cv2, cvs2, Smax, t_dev, single_launch=False)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    for a, b_ in zip(caches[0], caches[1]):
        assert torch.equal(a, b_), "appended cache rows differ"
    # one launch: the partials are merged in another order, so equal up to fp32 summation order; three calls in a
    # row check that the arrival counters are left ready for the next call
    for rep in range(3):
        ck3, cks3, cv3, cvs3 = (x.clone() for x in caches[0])
        ck3[:, t], cks3[:, t], cv3[:, t], cvs3[:, t] = 0, 0, 0, 0
        one = K.shared_prefix_attn_qkv(qkv, H, Hkv, D, cos, sin, pos_dev, pk if P else None, pv if P else None, P,
                                       ck3, cks3, cv3, cvs3, Smax, t_dev, single_launch=True)
        torch.cuda.synchronize()
        assert torch.allclose(one.float(), want.float(), rtol=2e-3, atol=2e-3), f"call {rep}: {float((one.float() - want.float()).abs().max())}"
        for a, b_ in zip(caches[0], (ck3, cks3, cv3, cvs3)):
            assert torch.equal(a, b_), "appended cache rows differ"


@pytest.mark.parametrize("B,H,Hkv,P,L", [(100, 4, 4, 150, 9), (33, 8, 2, 70, 4), (5, 4, 4, 0, 6), (128, 2, 2, 40, 0)])
def test_one_launch_attention_matches_two_launches(B, H, Hkv, P, L):
    """smh_shared_prefix_attn_one against smh_shared_prefix_attn on the same inputs (Q4_0 suffix, new token):
    same partials, merged in another order; called three times to check the counters are left ready."""
    from spec_mcts_amd import kernels as K
    dev = "cuda:0"
    D, Smax = 128, 16
    g = torch.Generator().manual_seed(1200 + B)
    q = (torch.randn((B, H, D), generator=g) * 0.7).half().to(dev)
    pk = (torch.randn((max(P, 1), Hkv, D), generator=g) * 0.5).half().to(dev)
    pv = (torch.randn((max(P, 1), Hkv, D), generator=g) * 0.5).half().to(dev)
    ck = torch.randint(-128, 128, (B, Smax, Hkv, 64), generator=g, dtype=torch.int16).to(torch.int8).to(dev)
    cv = torch.randint(-128, 128, (B, Smax, Hkv, 64), generator=g, dtype=torch.int16).to(torch.int8).to(dev)
    cks = (torch.rand((B, Smax, Hkv, 2), generator=g) * 0.1 + 0.01).half().to(dev)
    cvs = (torch.rand((B, Smax, Hkv, 2), generator=g) * 0.1 + 0.01).half().to(dev)
    k = (torch.randn((B, Hkv, D), generator=g) * 0.5).half().to(dev)
    v = (torch.randn((B, Hkv, D), generator=g) * 0.5).half().to(dev)
    lens = torch.tensor([L], dtype=torch.int32, device=dev)
    kw = dict(suffix_k=ck, suffix_v=cv, suffix_ks=cks, suffix_vs=cvs, Smax=Smax, lens=lens, lens_stride=0, cur_k=k, cur_v=v,
              n_kv_heads=Hkv)
    want = K.shared_prefix_attn(q, pk if P else None, pv if P else None, P, **kw)
    for rep in range(3):
        got = K.shared_prefix_attn(q, pk if P else None, pv if P else None, P, single_launch=True, **kw)
        torch.cuda.synchronize()
        assert torch.allclose(got.float(), want.float(), rtol=2e-3, atol=2e-3), f"call {rep}: {float((got.float() - want.float()).abs().max())}"
