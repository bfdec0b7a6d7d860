"""The kernels that Suranex brought, each against plain arithmetic, with inputs made so that a
fault shows: one key whose score stands out, placed at every edge a mask has."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_suranex as S
from kernel_refs import tile_cache
from yalis_amd.engine.batch import SeqSpan, attention_tiles, build_host_batch

pytestmark = pytest.mark.gpu

_ops = {}


def ops():
    if "o" not in _ops:
        from yalis_amd.ops.hip import HipOps

        _ops["o"] = HipOps("cuda:0")
    return _ops["o"]


def dense_attention(q, k, v, positions, heads_per_kv, scale, softcap, window, keep_first):
    """q [N, H, d] at ``positions``; k [L, G, d], v [L, G, dv] of one sequence: float64, a dense mask."""
    L = k.shape[0]
    mask = S.visible(L, window or L, keep_first)[positions]
    out = torch.empty(q.shape[0], q.shape[1], v.shape[2], dtype=torch.float64)
    for h in range(q.shape[1]):
        g = h // heads_per_kv
        s = (q[:, h].double() @ k[:, g].double().T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~mask, -float("inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g].double()
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("head_dim", [64, 128, 32])
@pytest.mark.parametrize("special", [400, 399, 69, 70, 63, 64, 0, 127, 128])
def test_one_key_stands_out_at_every_edge(dtype, head_dim, special):
    one_key_stands_out(dtype, head_dim, special, window=200, keep=70)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,keep,special", [(0, 0, 3), (0, 0, 321), (1000, 0, 5), (200, 0, 400), (200, 0, 401), (64, 64, 63), (64, 65, 64)])
def test_one_far_key_among_hundreds(dtype, window, keep, special):
    """No window at all (a far key among 700), a window larger than the sequence, a window without
    kept first keys, and kept first keys that end at a page's border."""
    one_key_stands_out(dtype, 64, special, window=window, keep=keep)


def one_key_stands_out(dtype, head_dim, special, window, keep):
    """A window of 200 keys with the first 70 kept, pages of 64: one key's score towers over the
    rest; a prompt's portion at positions 550..699 and single tokens at 599, 600, 269 and 270 look
    for it.  Key 400 leaves the window between 599 and 600, keys 69 / 70 are the last kept and the
    first not kept, 63 / 64 and 127 / 128 lie across borders of pages and key blocks."""
    o = ops()
    H, G, d, page, L = 4, 2, head_dim, 64, 700
    scale, softcap = 0.2, 30.0
    gen = torch.Generator().manual_seed(special)
    k = torch.randn(L, G, d, generator=gen) * 0.1
    v = torch.randn(L, G, d, generator=gen)
    k[special, :, 0] = 40.0
    k, v = k.to(dtype).float(), v.to(dtype).float()
    spans_at = [(550, 150), (599, 1), (600, 1), (269, 1), (270, 1)]
    n_pages = sum(-(-(p0 + n) // page) for p0, n in spans_at)
    perm = torch.randperm(n_pages, generator=gen).tolist()
    kc = torch.zeros(n_pages, G, page, d)
    vc = torch.zeros(n_pages, G, d, page)
    spans, used = [], 0
    for p0, n in spans_at:
        need = -(-(p0 + n) // page)
        table = np.array(perm[used: used + need], dtype=np.int32)
        used += need
        for j in range(p0 + n):
            kc[table[j // page], :, j % page] = k[j]
            vc[table[j // page], :, :, j % page] = v[j]
        spans.append(SeqSpan(tokens=[0] * n, first_position=p0, block_tables=[table], state_slot=len(spans), want=[]))
    hb = build_host_batch(spans, 1, page)
    positions = torch.from_numpy(hb.positions).long()
    q = torch.randn(hb.n_tokens, H, d, generator=gen) * 0.1
    q[:, :, 0] = 1.0
    q = q.to(dtype).float()
    want = dense_attention(q, k, v, positions, H // G, scale, softcap, window, keep)
    dev = "cuda:0"
    arrays = {"positions": torch.from_numpy(hb.positions).to(dev), "token_seq": torch.from_numpy(hb.token_seq).to(dev),
              "block_table_g0": torch.from_numpy(hb.block_tables[0]).to(dev)}
    ctx = SimpleNamespace(arrays=arrays, max_ctx=hb.max_ctx, host=hb)
    kc_d, vc_d = kc.to(dtype), vc.to(dtype)
    if o.masked_pages_tiled(dtype, d, d, page):
        kc_d, vc_d = tile_cache(kc_d, vc_d)
    kc_d, vc_d = kc_d.to(dev).contiguous(), vc_d.to(dev).contiguous()
    qd = q.to(dtype).reshape(hb.n_tokens, H * d).to(dev)
    tol = 2e-4 if dtype == torch.float32 else 4e-2
    got = o.attention_masked(qd, H, G, d, d, kc_d, vc_d, page, scale, ctx, 0, window=window, keep_first=keep, softcap=softcap)
    err = (got.float().cpu().view(-1, H, d).double() - want).abs().max(dim=2).values.max(dim=1).values
    assert err.max() < tol, f"general kernel: position {int(positions[int(err.argmax())])} differs by {err.max():.3e}"
    if dtype == torch.bfloat16 and d in (64, 128):
        tpt, big = o.attention_tokens_per_tile(H, G), o.attention_long_span_tile(H, G)
        tiles = torch.from_numpy(attention_tiles(hb, tpt, 1, big)).to(dev)
        long_tiles = torch.from_numpy(attention_tiles(hb, big, big + 1, longest_first=True)).to(dev)
        for plan, long_plan in ((None, None), ((4, 3), 2), ((1, 1), 1)):
            got = o.attention(qd, H, G, d, kc_d, vc_d, page, scale, window, ctx, 0, tiles, long_tiles, plan=plan, long_plan=long_plan,
                              keep_first=keep, softcap=softcap)
            err = (got.float().cpu().view(-1, H, d).double() - want).abs().max(dim=2).values.max(dim=1).values
            assert err.max() < tol, f"matrix cores, plan {plan}/{long_plan}: position {int(positions[int(err.argmax())])} differs by {err.max():.3e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,hidden,ff,experts,top", [
    (301, 32, 8, 1, 1), (301, 64, 8, 1, 1), (7, 64, 32, 4, 2), (70, 64, 32, 3, 1), (200, 64, 96, 2, 2), (500, 128, 64, 4, 2),
    (300, 96, 40, 2, 1), (33, 40, 24, 5, 3), (1, 128, 32, 8, 4), (640, 32, 32, 2, 2), (260, 256, 8, 1, 1), (130, 8, 8, 1, 1),
])
def test_experts_every_path(dtype, n, hidden, ff, experts, top):
    """The experts' rows against plain arithmetic at sizes that take every form of the two products:
    float32 FMA (any sizes), straight from memory into the matrix cores with tiles of 16 and of 64
    pairs, and tiles of 128 through LDS; widths down to 8, one expert, every expert chosen."""
    import kernel_refs as R

    gen = torch.Generator().manual_seed(n + hidden)
    x = torch.randn(n, hidden, generator=gen).to(dtype)
    ids = torch.randint(0, 50, (n,), generator=gen, dtype=torch.int32)
    table = torch.rand(50, experts, generator=gen).argsort(-1)[:, :top].to(torch.int32).contiguous()
    wgu = (torch.randn(experts, 2, ff, hidden, generator=gen) / hidden ** 0.5).to(dtype)
    wd = (torch.randn(experts, hidden, ff, generator=gen) / ff ** 0.5).to(dtype)
    act = ("clamped_swish", 1.5, 1.702)
    want = R.moe_experts(x, ids, table, wgu, wd, act)
    got = ops().moe_experts(x.cuda(), ids.cuda(), table.cuda(), wgu.cuda(), wd.cuda(), act).cpu()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    err = (got - want).abs().max(dim=1).values
    assert err.max() <= tol * max(1.0, float(want.abs().max())), f"row {int(err.argmax())} (token {int(err.argmax()) // top}) differs by {err.max():.3e}"
