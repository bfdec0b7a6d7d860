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


@pytest.mark.parametrize("head_dim,value_dim,page", [(64, 64, 64), (128, 128, 32), (32, 48, 16), (64, 64, 16)])
def test_qkv_prepare_forms_agree(head_dim, value_dim, page):
    """The form for many tokens (a head of eight tokens per workgroup, 16-byte stores) against the form
    for few (the same tokens in calls of 12) bit for bit, and both against plain arithmetic: norms,
    rotations and where everything lands in plain and tiled pages, for spans that start in the
    middle of a group of eight slots and for tokens of several requests."""
    import kernel_refs as R
    from yalis_amd.parts.base import Rotation

    o = ops()
    H, G, n = 4, 2, 60
    gen = torch.Generator().manual_seed(head_dim + page)
    cols = H * head_dim + G * (head_dim + value_dim) + 8
    qkv = torch.randn(n, cols, generator=gen).to(torch.bfloat16)
    # three requests: positions 3.., 0.. and 21..; their slots in pages of their own
    positions = torch.tensor(list(range(3, 28)) + list(range(0, 10)) + list(range(21, 46)), dtype=torch.int32)
    first_page = [0, 4, 6]
    owner = [0] * 25 + [1] * 10 + [2] * 25
    slots = torch.tensor([(first_page[r] + int(p) // page) * page + int(p) % page for r, p in zip(owner, positions)], dtype=torch.int32)
    n_pages = 6 + 46 // page + 2
    qn, kn = (1 + 0.3 * torch.randn(head_dim, generator=gen)).to(torch.bfloat16), (1 + 0.3 * torch.randn(head_dim, generator=gen)).to(torch.bfloat16)
    ang = torch.arange(64, dtype=torch.float32)[:, None] * (100.0 ** (-torch.arange(head_dim // 4, dtype=torch.float32) / (head_dim // 4)))
    rot = Rotation(torch.cos(ang).cuda(), torch.sin(ang).cuda(), head_dim // 2, False)
    vang = torch.arange(64, dtype=torch.float32)[:, None] * (100.0 ** (-torch.arange(value_dim // 2, dtype=torch.float32) / (value_dim // 2)))
    vrot = Rotation(torch.cos(vang).cuda(), torch.sin(vang).cuda(), value_dim, False)

    def run(chunks):
        k = torch.zeros(n_pages, G, page, head_dim, dtype=torch.bfloat16, device="cuda")
        v = torch.zeros(n_pages, G, value_dim, page, dtype=torch.bfloat16, device="cuda")
        qs = []
        for a, b in chunks:
            qs.append(o.qkv_prepare(qkv[a:b].cuda(), H, G, head_dim, value_dim, positions[a:b].cuda(), torch.bfloat16, q_norm=qn.cuda(),
                                    k_norm=kn.cuda(), qk_eps=1e-6, rotation=rot, value_norm_eps=1e-6, value_rotation=vrot,
                                    k_cache=k, v_cache=v, slots=slots[a:b].cuda(), page_size=page))
        return torch.cat(qs).cpu(), k.cpu(), v.cpu()

    many = run([(0, n)])
    few = run([(a, min(a + 12, n)) for a in range(0, n, 12)])
    for a, b, what in zip(many, few, ("queries", "key pages", "value pages")):
        assert torch.equal(a, b), f"{what} differ between the two forms"
    k_ref = torch.zeros(n_pages, G, page, head_dim, dtype=torch.bfloat16)
    v_ref = torch.zeros(n_pages, G, value_dim, page, dtype=torch.bfloat16)
    cpu = lambda r: Rotation(r.cos.cpu(), r.sin.cpu(), r.rotary_dim, r.interleaved)
    q_ref = R.qkv_prepare(qkv, H, G, head_dim, value_dim, positions, torch.bfloat16, q_norm=qn, k_norm=kn, qk_eps=1e-6, rotation=cpu(rot),
                          value_norm_eps=1e-6, value_rotation=cpu(vrot), k_cache=k_ref, v_cache=v_ref, slots=slots, page_size=page)
    k_got, v_got = many[1], many[2]
    if o.masked_pages_tiled(torch.bfloat16, head_dim, value_dim, page):
        from kernel_refs import untile_cache

        k_got, v_got = untile_cache(k_got, v_got)
    assert (many[0].float() - q_ref.float()).abs().max() <= 0.04
    assert (k_got.float() - k_ref.float()).abs().max() <= 0.04 and (v_got.float() - v_ref.float()).abs().max() <= 0.04
