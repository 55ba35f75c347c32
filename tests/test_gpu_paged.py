"""Tree (paged) attention and the page-table fork: suffix rows are looked up through a page table inside the kernel, so
branches forked from a common ancestor share its rows.  The generators mirror the reference's own checks
(triton_kernels_bench.py:369-403 rand_paged_qkv, :433-475 branch_paged_qkv: N(0, 0.5) values, one fork per step until
B branches exist; its check is page_flash_attn against F.scaled_dot_product_attention at atol 1e-2, :479-493); the
values come from a CPU generator, since the reference's CUDA random streams cannot be reproduced."""
import pytest
import torch
import torch.nn.functional as F

from oracle import q40_oracle as O
from tests.sync_state import sync_prefix, sync_suffix_row

pytestmark = pytest.mark.gpu


def branch_paged(B, L, H, D, prompt_L, seed, dtype=torch.int16):
    """A tree of B branches over L positions: all share the prompt's pages; at every step after the prompt one more
    branch forks from the previous one (sharing all its pages so far), then every live branch gets a new page."""
    g = torch.Generator().manual_seed(seed)
    q = torch.empty((B, H, D)).normal_(0.0, 0.5, generator=g).half()
    pager = torch.zeros((B, L), dtype=torch.int64)
    pager[:, :prompt_L] = torch.arange(prompt_L)
    page_idx, b = prompt_L, 1
    for i in range(prompt_L, L):
        if b < B:
            pager[b, :i] = pager[b - 1, :i]
            b += 1
        pager[:b, i] = page_idx + torch.arange(b)
        page_idx += b
    P = 1
    while P <= page_idx:
        P *= 2
    k_pages = torch.empty((H, P, D)).normal_(0.0, 0.5, generator=g).half()
    v_pages = torch.empty((H, P, D)).normal_(0.0, 0.5, generator=g).half()
    return P, q, pager.to(dtype), k_pages, v_pages


def sdpa(q, pager, k_pages, v_pages, lens=None):
    """F.scaled_dot_product_attention over the gathered dense K/V (the reference's oracle for this operator)."""
    B, L = pager.shape
    out = torch.empty((B,) + tuple(q.shape[1:]))
    for b in range(B):
        n = L if lens is None else int(lens[b])
        idx = pager[b, :n].long()
        k = k_pages[:, idx].float()                     # [H, n, D]
        v = v_pages[:, idx].float()
        out[b] = F.scaled_dot_product_attention(q[b].float()[:, None], k, v)[:, 0]
    return out


def test_tree_attention_on_the_reference_check_shape():
    from spec_mcts_amd import kernels as K
    B, L, H, D, prompt_L = 27, 512, 32, 128, 256
    P, q, pager, kp, vp = branch_paged(B, L, H, D, prompt_L, seed=1)
    assert pager.dtype == torch.int16 and int(pager.max()) < P
    # the tree really shares pages beyond the prompt
    assert torch.equal(pager[26, prompt_L:prompt_L + 20], pager[25, prompt_L:prompt_L + 20]) and not torch.equal(pager[26, 300:], pager[25, 300:])
    want = sdpa(q, pager, kp, vp)
    got = K.page_flash_attn(pager.cuda(), q.cuda(), kp.cuda(), vp.cuda(), P, B, L, H, D).cpu().float()
    assert torch.allclose(got, want, atol=1e-2, rtol=0), float((got - want).abs().max())
    assert bool(((got - want).abs() <= 2e-3 + 1e-2 * want.abs()).all())
    # the shared chunk as the kernel's prefix (staged once for all branches), the rest through the page table
    got_c = K.chunk_attn(pager.cuda(), q.cuda(), kp.cuda(), vp.cuda(), P, B, L, H, D, prompt_L).cpu().float()
    assert torch.allclose(got_c, want, atol=1e-2, rtol=0)


@pytest.mark.parametrize("B", [1, 2, 7, 64, 99])
def test_tree_attention_every_branch_count(B):
    """the reference sweeps every B in 1..99 (triton_kernels_bench.py:541-547); a spread of them here, shorter sequences"""
    from spec_mcts_amd import kernels as K
    L, H, D, prompt_L = 160, 8, 128, 96
    P, q, pager, kp, vp = branch_paged(B, L, H, D, prompt_L, seed=10 + B, dtype=torch.int32)
    want = sdpa(q, pager, kp, vp)
    got = K.page_flash_attn(pager.cuda(), q.cuda(), kp.cuda(), vp.cuda(), P, B, L, H, D).cpu().float()
    assert torch.allclose(got, want, atol=1e-2, rtol=0)


@pytest.mark.parametrize("dtype", [torch.int16, torch.int32, torch.int64])
@pytest.mark.parametrize("single_launch", [False, True])
def test_paged_q40_pool_ragged_lengths_and_current_token(dtype, single_launch):
    """The model's form: token-major Q4_0 rows + scales as the pool, a token-major fp16 prefix, ragged numbers of valid
    pages per branch, grouped-query heads, the new token's exact fp16 K/V; page ids of 2, 4 and 8 bytes; both launch forms."""
    from spec_mcts_amd import kernels as K
    B, H, Hkv, D, Pfx, S, rows = 6, 8, 2, 128, 70, 40, 300
    g = torch.Generator().manual_seed(77)
    q = torch.randn((B, H, D), generator=g).half()
    pk, pv = torch.randn((Pfx, Hkv, D), generator=g).half(), torch.randn((Pfx, Hkv, D), generator=g).half()
    pool_k, pool_v = torch.randn((rows, Hkv, D), generator=g).half(), torch.randn((rows, Hkv, D), generator=g).half()
    kw, ks = O.quantize_q40(pool_k, 64)
    vw, vs = O.quantize_q40(pool_v, 64)
    dk = O.dequantize_q40(kw, ks, 64, pool_k.shape)
    dv = O.dequantize_q40(vw, vs, 64, pool_v.shape)
    pages = torch.randint(0, rows, (B, S), generator=g).to(dtype)          # arbitrary sharing: any branch may name any row
    lens = torch.tensor([0, 1, 40, 17, 33, 5], dtype=torch.int32)
    ck, cv = torch.randn((B, Hkv, D), generator=g).half(), torch.randn((B, Hkv, D), generator=g).half()
    sk = torch.zeros((B, S + 1, Hkv, D), dtype=torch.float16)
    sv = torch.zeros((B, S + 1, Hkv, D), dtype=torch.float16)
    for b in range(B):
        n = int(lens[b])
        sk[b, :n], sv[b, :n] = dk[pages[b, :n].long()], dv[pages[b, :n].long()]
        sk[b, n], sv[b, n] = ck[b], cv[b]
    want = O.shared_prefix_attention(q, pk, pv, sk, sv, [int(x) + 1 for x in lens]).float()
    got = K.paged_prefix_attn(q.cuda(), pages.cuda(), lens.cuda(), kw.view(rows, Hkv, 64).cuda(), vw.view(rows, Hkv, 64).cuda(),
                              ks.view(rows, Hkv, 2).cuda(), vs.view(rows, Hkv, 2).cuda(), prefix_k=pk.cuda(), prefix_v=pv.cuda(), P=Pfx,
                              cur_k=ck.cuda(), cur_v=cv.cuda(), single_launch=single_launch).cpu().float()
    assert bool(((got - want).abs() <= 2e-3 + 1e-2 * want.abs()).all()), float((got - want).abs().max())
    # identity page table = the contiguous-rows entry point, bit for bit
    ident = (torch.arange(B)[:, None] * S + torch.arange(S)[None]).to(dtype)
    a = K.paged_prefix_attn(q.cuda(), ident.cuda(), lens.cuda(), kw.view(rows, Hkv, 64)[:B * S].contiguous().cuda(), vw.view(rows, Hkv, 64)[:B * S].contiguous().cuda(),
                            ks.view(rows, Hkv, 2)[:B * S].contiguous().cuda(), vs.view(rows, Hkv, 2)[:B * S].contiguous().cuda(), prefix_k=pk.cuda(), prefix_v=pv.cuda(),
                            P=Pfx, cur_k=ck.cuda(), cur_v=cv.cuda(), single_launch=single_launch)
    b_ = K.shared_prefix_attn(q.cuda(), pk.cuda(), pv.cuda(), Pfx, suffix_k=kw.view(rows, Hkv, 64)[:B * S].contiguous().cuda(),
                              suffix_v=vw.view(rows, Hkv, 64)[:B * S].contiguous().cuda(), suffix_ks=ks.view(rows, Hkv, 2)[:B * S].contiguous().cuda(),
                              suffix_vs=vs.view(rows, Hkv, 2)[:B * S].contiguous().cuda(), Smax=S, lens=lens.cuda(), lens_stride=1,
                              cur_k=ck.cuda(), cur_v=cv.cuda(), single_launch=single_launch)
    assert torch.equal(a, b_)


def test_page_ids_outside_the_pool_read_the_nearest_row():
    """A page id below 0 or past the pool (a corrupted table) is read as row 0 or the last row: the affected branch's
    result is that of the cut table, bit for bit, and nothing outside the pool is touched."""
    from spec_mcts_amd import kernels as K
    B, H, Hkv, D, S, rows = 4, 4, 2, 128, 24, 64
    g = torch.Generator().manual_seed(78)
    q = torch.randn((B, H, D), generator=g).half()
    kw, ks = O.quantize_q40(torch.randn((rows, Hkv, D), generator=g).half(), 64)
    vw, vs = O.quantize_q40(torch.randn((rows, Hkv, D), generator=g).half(), 64)
    pages = torch.randint(0, rows, (B, S), generator=g).to(torch.int32)
    bad = pages.clone()
    bad[1, 3], bad[2, 0], bad[3, 20] = -7, rows + 1000, 2 ** 30
    lens = torch.tensor([24, 24, 10, 21], dtype=torch.int32)
    args = (kw.view(rows, Hkv, 64).cuda(), vw.view(rows, Hkv, 64).cuda(), ks.view(rows, Hkv, 2).cuda(), vs.view(rows, Hkv, 2).cuda())
    got = K.paged_prefix_attn(q.cuda(), bad.cuda(), lens.cuda(), *args)
    want = K.paged_prefix_attn(q.cuda(), bad.clamp(0, rows - 1).cuda(), lens.cuda(), *args)
    assert torch.equal(got, want) and bool(torch.isfinite(got.float()).all())


def test_page_fork_copies_page_ids():
    from spec_mcts_amd import kernels as K
    table = torch.arange(8 * 300, dtype=torch.int32).view(8, 300).cuda()
    want = table.clone()
    K.page_fork(table, 1, 4, 3, 257)
    want[4:7, :257] = want[1, :257]
    assert torch.equal(table, want)
    K.page_fork(table, 0, 7, 1, 0)                      # nothing written yet: nothing to copy
    assert torch.equal(table, want)
    from spec_mcts_amd import _lib
    with pytest.raises(_lib.SmhError):
        K.page_fork(table, 5, 4, 3, 10)                 # origin inside the destination rows


SMALL = dict(dim=256, n_layers=2, n_heads=2, vocab_size=320, multiple_of=128, max_batch_size=8, max_seq_len=24,
             max_prompt_seq_len=32)
GQA = dict(dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=384, multiple_of=128, max_batch_size=24,
           max_seq_len=16, max_prompt_seq_len=48)


@pytest.mark.parametrize("cfg,seed,fused", [(SMALL, 50, True), (GQA, 51, True), (SMALL, 52, False)])
def test_fork_heavy_decode_matches_oracle_and_row_copy(cfg, seed, fused):
    """A tree grown the way mcts.search grows it (mcts.py:127-152): forks of several origins, some of them themselves
    forked earlier, at every other step, each branch fed its own token.  The page-table fork (nothing copied) must give
    the logits of the oracle's row-copy fork and of this package's own row-copy path."""
    from spec_mcts_amd import ModelArgs
    from spec_mcts_amd.load_q40 import load_q40
    oargs = O.OracleArgs(**cfg)
    sd = O.random_q40_state_dict(oargs, seed=seed, std=0.05)
    oracle = O.OracleTransformer(oargs, sd, dense=True)
    models = {}
    for paged in (True, False):
        m = load_q40(dict(sd), ModelArgs(**cfg), device="cuda:0")
        m.paged_kv, m.fused = paged, fused
        models[paged] = m
    g = torch.Generator().manual_seed(seed + 100)
    P = 13
    prompt = torch.randint(0, cfg["vocab_size"], (1, P), generator=g)
    oracle.forward(prompt, 0)
    for m in models.values():
        m(prompt.cuda(), 0)
        sync_prefix(m, oracle)
    Bmax = cfg["max_batch_size"]
    live = 1
    plan = {2: [(0, 2)], 4: [(1, 1), (0, 1)], 5: [(3, 2)], 7: [(2, 1), (5, 10 ** 6)]}      # step -> (origin, forks) in order
    for s in range(9):
        for origin, forks in plan.get(s, []):
            forks = min(forks, Bmax - live)
            if origin < live and forks > 0:
                oracle.fork(origin, live, forks)
                for m in models.values():
                    m.fork(origin, live, forks)
                live += forks
        tok = torch.randint(0, cfg["vocab_size"], (live, 1), generator=g)                    # every branch its own token
        want = oracle.forward(tok, P + s)[:, -1].float()
        got = {paged: m(tok.cuda(), P + s)[:, -1].float().cpu() for paged, m in models.items()}
        assert torch.equal(got[True], got[False]), f"step {s}: the page-table fork differs from the row-copy fork"
        assert torch.allclose(got[True], want, rtol=2e-2, atol=2e-2), f"step {s}: max diff {float((got[True] - want).abs().max())}"
        for m in models.values():
            sync_suffix_row(m, oracle, live, s)        # every step starts from the oracle's cache state
    assert live > 6 and models[True]._forked
    # a new prompt starts from unshared rows again
    models[True].resetSeq()
    assert models[True]._pages(torch.device("cuda:0")) is None


def test_lens_are_cut_to_the_columns_of_a_sliced_table():
    """a column slice of a wider page table: the rows are `stride` apart but hold fewer ids; a length beyond the slice is cut
    to it inside the kernel (no id of the next columns, or past the last row's end, is read)"""
    from spec_mcts_amd import kernels as K
    B, L, H, D, prompt_L = 9, 96, 4, 128, 32
    P, q, pager, kp, vp = branch_paged(B, L, H, D, prompt_L, seed=77, dtype=torch.int32)
    off, cols = 40, 30
    table = pager.cuda()
    view = table[:, off:off + cols]                                  # stride L, 30 ids a row
    assert view.stride(0) == L and view.shape[1] == cols
    over = torch.full((B,), 10 * L, dtype=torch.int32, device="cuda")
    got = K.paged_prefix_attn(q.cuda(), view, over, kp.cuda(), vp.cuda(), head_major=True).cpu().float()
    want = sdpa(q, pager[:, off:off + cols], kp, vp)
    assert torch.allclose(got, want, atol=1e-2, rtol=0)
    # the last row's slice ends before the table does; with the slice at the very end of the table the cut is what keeps
    # the reads inside it
    tail = table[:, L - cols:]
    got = K.paged_prefix_attn(q.cuda(), tail, over, kp.cuda(), vp.cuda(), head_major=True).cpu().float()
    want = sdpa(q, pager[:, L - cols:], kp, vp)
    assert torch.allclose(got, want, atol=1e-2, rtol=0)
