"""Tiled weight layout (smh_q40_tile, smh_q40_matmul_partial_tiled): the tiles against an element-by-element
numpy statement of the layout, and the products against the checkpoint-layout kernels (bit for bit) and the oracle."""
import numpy as np
import pytest
import torch

from oracle import q40_oracle as O

pytestmark = pytest.mark.gpu

TILE_W, TILE_S = 4096, 256
TILE = TILE_W + TILE_S


def tiles_by_definition(w: np.ndarray, s: np.ndarray, K: int, N: int) -> np.ndarray:
    """w uint8 [K, N/2], s uint16 [K, N/64] -> uint8 [units, steps, 4352].  Every checkpoint byte (k, byte column)
    goes to: unit = column / 128, blk = column % 128 / 64, c = column % 64 / 4, B = column % 4, step = k / 32,
    g = k % 32 / 8, i = k % 8; piece 2 blk + B / 2, lane 16 g + c, dword 2 (B % 2) + [i in 2,3,6,7], byte
    (0, 2, 0, 2, 1, 3, 1, 3)[i]; value XOR 0x88.  Scale (k, group G): unit G / 4, offset 4096 + 16 (4 g + G % 4) + 2 i."""
    units, steps = (N + 255) // 256, (K + 31) // 32
    out = np.zeros((units, steps, TILE), dtype=np.uint8)
    out[:, :, :TILE_W] = 0x88
    k, col = np.meshgrid(np.arange(K), np.arange(N // 2), indexing="ij")
    unit, blk, c, B = col // 128, col % 128 // 64, col % 64 // 4, col % 4
    step, g, i = k // 32, k % 32 // 8, k % 8
    dword = 2 * (B % 2) + np.isin(i, (2, 3, 6, 7)).astype(np.int64)
    byte = np.array([0, 2, 0, 2, 1, 3, 1, 3])[i]
    off = (2 * blk + B // 2) * 1024 + (16 * g + c) * 16 + dword * 4 + byte
    out[unit, step, off] = w ^ 0x88
    k, G = np.meshgrid(np.arange(K), np.arange(N // 64), indexing="ij")
    off = TILE_W + 16 * (4 * (k % 32 // 8) + G % 4) + 2 * (k % 8)
    s8 = s.view(np.uint8).reshape(K, N // 64, 2)
    out[G // 4, k // 32, off] = s8[:, :, 0]
    out[G // 4, k // 32, off + 1] = s8[:, :, 1]
    return out


def _weight(K, N, seed):
    g = torch.Generator().manual_seed(seed)
    v = (torch.randn((N, K), generator=g) * 0.02).half()
    w, s, _ = O.quantize_weight(v)
    return w, s


@pytest.mark.parametrize("K,N", [(32, 128), (64, 256), (40, 384), (256, 640), (4096, 512)])
def test_tiles_match_the_layout_definition(K, N):
    from spec_mcts_amd import kernels as Kn
    w, s = _weight(K, N, 900 + K + N)
    t = Kn.tile_q40(w.cuda(), s.cuda(), K, N)
    got = t.buf.cpu().numpy().reshape((N + 255) // 256, (K + 31) // 32, TILE)
    want = tiles_by_definition(w.numpy().view(np.uint8).reshape(K, N // 2), s.numpy().view(np.uint16).reshape(K, N // 64), K, N)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("M", [1, 3, 10, 16, 17, 65, 100, 128, 130])
@pytest.mark.parametrize("K,ns", [(64, [128]), (40, [384]), (4096, [4096]), (1000, [256, 128, 128]), (4096, [1024, 256, 256]),
                                  (11008, [4096]), (4096, [11008, 11008]),
                                  # 1, 3, 5 and 7 steps of 32 rows: the ends of a loop that takes its steps in pairs
                                  (32, [128]), (96, [256]), (160, [128]), (224, [384]), (416, [256])])
def test_tiled_products_equal_checkpoint_layout_products(M, K, ns):
    """same operands into the same MFMAs in the same order: the slabs are bit-identical wherever the two layouts share a
    plan (always up to 16 rows, above 128 rows and when K is not a multiple of 64; between, tiled weights may run the
    kernel with two K-groups a workgroup, which leaves fewer slabs); both against the oracle's matmul in every case"""
    from spec_mcts_amd import kernels as Kn
    ws = [_weight(K, n, 910 + i + K) for i, n in enumerate(ns)]
    a = (torch.randn((M, K), generator=torch.Generator().manual_seed(920 + M)) * 0.5).half().cuda()
    lin = [(w.cuda(), s.cuda(), n) for (w, s), n in zip(ws, ns)]
    tiled = [Kn.tile_q40(w, s, K, n) for (w, s, n) in lin]
    p0 = Kn.matmul_q40_partial(a, lin)
    p1 = Kn.matmul_q40_partial(a, tiled)
    torch.cuda.synchronize()
    assert p0.n_total == p1.n_total and p1.ksplit == Kn.matmul_plan(M, K, ns, tiled=True) and p0.ksplit == Kn.matmul_plan(M, K, ns)
    if not (16 < M <= 128 and K % 64 == 0):
        assert p0.ksplit == p1.ksplit
        n = p0.ksplit * M * p0.n_total            # fp32 slabs at every batch size
        assert torch.equal(p0.buf[:n].view(torch.int32), p1.buf[:n].view(torch.int32))
    # and against the oracle's matmul (fp32 accumulation of the dequantised matrix)
    for p in (p0, p1):
        got = Kn.partial_reduce(p).cpu()
        col = 0
        for (w, s), nn in zip(ws, ns):
            want = O.matmul_q40(a.cpu(), w, s, (K, nn))
            assert torch.allclose(got[:, col:col + nn].float(), want.float(), rtol=1e-2, atol=2e-3)
            col += nn


@pytest.mark.parametrize("M", [17, 100, 128])
@pytest.mark.parametrize("K,ns,slabs", [(4096, [11008, 11008], 4), (2048, [16640, 16640], 3), (1024, [7680, 7680, 7680], 4)])
def test_range_cut_products(M, K, ns, slabs):
    """launches whose even split would put two workgroups on some compute units and one on others deal runs of steps
    instead: a workgroup may end one column unit and begin the next (also across two weights of the launch), and a unit
    with fewer pieces than slabs gets zeros for the rest.  Slab count as planned, slabs equal in both layouts bit for
    bit where tiled weights take the same plan (up to 64 rows, or more column blocks than compute units), sums against the
    oracle in both layouts."""
    from spec_mcts_amd import kernels as Kn
    assert Kn.matmul_plan(M, K, ns) == slabs
    slabs_tiled = Kn.matmul_plan(M, K, ns, tiled=True)
    assert slabs_tiled == slabs or (M > 64 and slabs_tiled < slabs)
    ws = [_weight(K, n, 960 + i + K) for i, n in enumerate(ns)]
    a = (torch.randn((M, K), generator=torch.Generator().manual_seed(970 + M)) * 0.5).half().cuda()
    lin = [(w.cuda(), s.cuda(), n) for (w, s), n in zip(ws, ns)]
    tiled = [Kn.tile_q40(w, s, K, n) for (w, s, n) in lin]
    # slabs full of NaNs before the launch: a column no piece or zero fill writes would show
    n = slabs * M * sum(ns)
    out0 = torch.full((n,), float("nan"), dtype=torch.float32, device="cuda")
    out1 = out0.clone()
    p0 = Kn.matmul_q40_partial(a, lin, out0)
    p1 = Kn.matmul_q40_partial(a, tiled, out1)
    torch.cuda.synchronize()
    assert p0.ksplit == slabs and p1.ksplit == slabs_tiled
    n1 = slabs_tiled * M * sum(ns)
    assert not torch.isnan(p0.buf[:n]).any() and not torch.isnan(p1.buf[:n1]).any()
    if slabs_tiled == slabs:
        assert torch.equal(p0.buf[:n].view(torch.int32), p1.buf[:n].view(torch.int32))
    for p in (p0, p1):
        got = Kn.partial_reduce(p).cpu()
        col = 0
        for (w, s), nn in zip(ws, ns):
            want = O.matmul_q40(a.cpu(), w, s, (K, nn))
            assert torch.allclose(got[:, col:col + nn].float(), want.float(), rtol=1e-2, atol=2e-3)
            col += nn


@pytest.mark.parametrize("M", [17, 33, 64, 100, 128])
@pytest.mark.parametrize("K,n_half", [(4096, 11008), (256, 384), (8192, 1024), (128, 128), (1024, 16384)])
def test_swiglu_inside_the_gate_up_launch(M, K, n_half):
    """smh_q40_matmul_tiled_swiglu (hf_model_q40_kv_shared.py:434, `F.silu(self.w1(x)) * self.w3(x)`) against the oracle's two
    linears, SiLU and product with their fp16 roundings, and against the two launches it replaces (smh_q40_matmul_partial_tiled
    + smh_partial_silu_mul: the same roundings, another order of the fp32 additions, so single fp16 ulps may differ)"""
    import torch.nn.functional as F
    from spec_mcts_amd import kernels as Kn
    w1, w3 = _weight(K, n_half, 980 + K), _weight(K, n_half, 981 + K)
    x = (torch.randn((M, K), generator=torch.Generator().manual_seed(982 + M)) * 0.5).half()
    t1, t3 = Kn.tile_q40(w1[0].cuda(), w1[1].cuda(), K, n_half), Kn.tile_q40(w3[0].cuda(), w3[1].cuda(), K, n_half)
    got = Kn.matmul_q40_swiglu(x.cuda(), t1, t3)
    two = Kn.partial_silu_mul(Kn.matmul_q40_partial(x.cuda(), [t1, t3]))
    torch.cuda.synchronize()
    g16, u16 = O.matmul_q40(x, w1[0], w1[1], (K, n_half)), O.matmul_q40(x, w3[0], w3[1], (K, n_half))
    want = F.silu(g16.float()).half() * u16
    assert got.shape == (M, n_half) and got.dtype == torch.float16
    assert torch.allclose(got.cpu().float(), want.float(), rtol=1e-2, atol=2e-3)
    assert torch.allclose(got.float(), two.float(), rtol=4e-3, atol=1e-4)
    assert float((got != two).float().mean()) < 0.02
    assert Kn.swiglu_fits(M, K, n_half) == (M > 32 and n_half >= 8192)


def test_model_logits_do_not_depend_on_the_weight_layout():
    """the fused forward on tiled copies against the same forward on the checkpoint tensors: equal bit for bit,
    at prefill (GEMM), at decode (GEMV) and again after a weight has been replaced"""
    from spec_mcts_amd import ModelArgs
    from spec_mcts_amd.load_q40 import load_q40
    cfg = dict(dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=384, multiple_of=128, max_batch_size=4,
               max_seq_len=16, max_prompt_seq_len=48)
    oargs = O.OracleArgs(**cfg)
    sd = O.random_q40_state_dict(oargs, seed=941)
    model = load_q40(dict(sd), ModelArgs(**cfg), device="cuda:0")
    prompt = torch.randint(0, cfg["vocab_size"], (1, 37), generator=torch.Generator().manual_seed(942)).cuda()
    tok = torch.randint(0, cfg["vocab_size"], (3, 1), generator=torch.Generator().manual_seed(943)).cuda()

    def run():
        model.resetSeq()
        return [model(prompt, 0).clone(), model(tok, 37).clone(), model(tok, 38).clone()]

    assert model.tiled_weights
    a = run()
    model.tiled_weights = False
    b = run()
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    # a replaced weight is re-tiled on the next use
    lin = model.layers[1].feed_forward.w2
    lin.w = lin.w.roll(1, 0).contiguous()
    lin.s = lin.s.roll(3).contiguous()
    c = run()
    model.tiled_weights = True
    d = run()
    assert not torch.equal(c[1], b[1])
    for x, y in zip(c, d):
        assert torch.equal(x, y)


@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("K,n1,n2", [(11008, 4096, 4096), (256, 128, 512), (2048, 384, 256), (28672, 8192, 1024)])
def test_w2_that_makes_its_own_silu_activations(M, K, n1, n2):
    """smh_q40_matmul_partial_tiled_silu against smh_partial_silu_mul + smh_q40_matmul_partial_tiled: bit-identical slabs
    (K = FFN width, n1 = model width feeding w1|w3, n2 = columns of w2)"""
    from spec_mcts_amd import kernels as Kn
    w1, w3, w2 = _weight(n1, K, 950 + K), _weight(n1, K, 951 + K), _weight(K, n2, 952 + K)
    x = (torch.randn((M, n1), generator=torch.Generator().manual_seed(953 + M)) * 0.7).half().cuda()
    t1, t3 = Kn.tile_q40(w1[0].cuda(), w1[1].cuda(), n1, K), Kn.tile_q40(w3[0].cuda(), w3[1].cuda(), n1, K)
    t2 = Kn.tile_q40(w2[0].cuda(), w2[1].cuda(), K, n2)
    gu = Kn.matmul_q40_partial(x, [t1, t3])
    want = Kn.matmul_q40_partial(Kn.partial_silu_mul(gu), [t2])
    got = Kn.matmul_q40_partial_silu(gu, [t2])
    torch.cuda.synchronize()
    n = want.ksplit * M * want.n_total
    assert got.ksplit == want.ksplit
    assert torch.equal(got.buf[:n].view(torch.int32), want.buf[:n].view(torch.int32))


@pytest.mark.parametrize("M", [1, 2, 7, 10, 16])
@pytest.mark.parametrize("n0,K,ns", [(1024, 4096, (4096, 1024, 1024)), (256, 4096, (11008, 11008)), (384, 512, (384,)),
                                     (512, 8192, (1024, 256)), (256, 1152, (128, 256))])
def test_matmul_that_makes_its_own_rmsnorm(M, n0, K, ns):
    """smh_partial_residual_sumsq + smh_q40_matmul_partial_tiled_norm against smh_partial_rmsnorm +
    smh_q40_matmul_partial_tiled on the slabs of a first matmul (n0 -> K) and a residual: the same residual stream and
    the same slabs, bit for bit, wherever the library says the shape fits."""
    from spec_mcts_amd import kernels as Kn
    g = torch.Generator().manual_seed(960 + M + K)
    w0 = _weight(n0, K, 961 + K)
    t0 = Kn.tile_q40(w0[0].cuda(), w0[1].cuda(), n0, K)
    ops = []
    for i, n in enumerate(ns):
        w = _weight(K, n, 962 + K + i)
        ops.append(Kn.tile_q40(w[0].cuda(), w[1].cuda(), K, n))
    x = (torch.randn((M, n0), generator=g) * 0.8).half().cuda()
    resid = torch.randn((M, K), generator=g).half().cuda()
    norm_w = (1.0 + 0.2 * torch.randn(K, generator=g)).half().cuda()
    eps = 1e-5
    first = Kn.matmul_q40_partial(x, [t0])
    h_want, xn = Kn.partial_rmsnorm(first, resid, norm_w, eps)
    want = Kn.matmul_q40_partial(xn, ops)
    if not Kn.norm_in_fits(M, K, list(ns)):
        h, sums = Kn.partial_residual_sumsq(first, resid)
        with pytest.raises(RuntimeError, match="K-slices"):
            Kn.matmul_q40_partial_norm(h, sums, norm_w, eps, ops)
        return
    h, sums = Kn.partial_residual_sumsq(first, resid)
    got = Kn.matmul_q40_partial_norm(h, sums, norm_w, eps, ops)
    torch.cuda.synchronize()
    assert torch.equal(h, h_want)
    # the sums of squares, added in index order in fp32, against fp64 of the same row
    ref = (h.double() ** 2).sum(1)
    tot = sums.double().sum(1)
    assert torch.allclose(tot, ref, rtol=1e-5)
    n = want.ksplit * M * want.n_total
    assert got.ksplit == want.ksplit
    assert torch.equal(got.buf[:n].view(torch.int32), want.buf[:n].view(torch.int32))


def test_rmsnorm_in_matmul_shape_limits():
    """the 70B-architecture w1|w3 launch holds one row's K-slice (4096 of 8192) but not ten; M above 16 never fits"""
    from spec_mcts_amd import kernels as Kn
    assert Kn.norm_in_fits(1, 8192, [28672, 28672])
    assert not Kn.norm_in_fits(10, 8192, [28672, 28672])
    assert Kn.norm_in_fits(16, 4096, [11008, 11008])
    assert not Kn.norm_in_fits(17, 4096, [4096])


def test_model_logits_do_not_depend_on_where_rmsnorm_is_made():
    """the fused forward with RMSNorm inside the matmuls against the same forward with partial_rmsnorm launches: equal bit
    for bit at decode with 1, 3 and 4 branches"""
    from spec_mcts_amd import ModelArgs
    from spec_mcts_amd.load_q40 import load_q40
    cfg = dict(dim=512, n_layers=3, n_heads=4, n_kv_heads=2, vocab_size=384, multiple_of=128, max_batch_size=4,
               max_seq_len=16, max_prompt_seq_len=48)
    oargs = O.OracleArgs(**cfg)
    sd = O.random_q40_state_dict(oargs, seed=971)
    model = load_q40(dict(sd), ModelArgs(**cfg), device="cuda:0")
    prompt = torch.randint(0, cfg["vocab_size"], (1, 21), generator=torch.Generator().manual_seed(972)).cuda()
    for B in (1, 3, 4):
        tok = torch.randint(0, cfg["vocab_size"], (B, 1), generator=torch.Generator().manual_seed(973 + B)).cuda()

        def run():
            model.resetSeq()
            return [model(prompt, 0).clone(), model(tok, 21).clone(), model(tok, 22).clone()]

        model.norm_in_matmul, model.norm_in_max_rows = True, 16
        a = run()
        assert model._norm_in_ok and all(model._norm_in_ok.values())
        model.norm_in_matmul = False
        b = run()
        for x, y in zip(a, b):
            assert torch.equal(x, y)
