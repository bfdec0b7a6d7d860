"""The kernels that Nutavik brought, each against plain arithmetic (tests/kernel_refs.py, float64
where the inputs are made by hand), at sizes of their own, odd ones included, and with inputs made so
that a fault shows: one page row whose score stands out, placed at every border."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import kernel_refs as R
from yalis_amd.engine.batch import SeqSpan, attention_tiles, build_host_batch
from yalis_amd.parts.base import Rotation

pytestmark = pytest.mark.gpu

_ops = {}


def ops():
    if "o" not in _ops:
        from yalis_amd.ops.hip import HipOps

        _ops["o"] = HipOps("cuda:0")
    return _ops["o"]


def context(spans_at, page, slots=None, tile_tokens=4, device="cuda:0"):
    """A step's integer arrays for requests that bring ``n`` tokens from position ``p0`` on (pages dealt
    out in a shuffled order); returns (ctx on the device, ctx on the CPU, pages used)."""
    gen = torch.Generator().manual_seed(len(spans_at))
    n_pages = sum(-(-(p0 + n) // page) for p0, n in spans_at)
    perm = torch.randperm(n_pages, generator=gen).tolist()
    spans, used = [], 0
    for i, (p0, n) in enumerate(spans_at):
        need = -(-(p0 + n) // page)
        spans.append(SeqSpan(tokens=[0] * n, first_position=p0, block_tables=[np.array(perm[used: used + need], dtype=np.int32)],
                             state_slot=i if slots is None else slots[i], want=[]))
        used += need
    hb = build_host_batch(spans, 1, page)
    arrays = {"positions": hb.positions, "token_seq": hb.token_seq, "seq_qstart": hb.seq_qstart, "seq_qlen": hb.seq_qlen,
              "state_slots": hb.state_slots, "block_table_g0": hb.block_tables[0], "slots_g0": hb.slots[0],
              f"latent_tiles_{tile_tokens}": attention_tiles(hb, tile_tokens)}
    cpu = SimpleNamespace(arrays={k: torch.from_numpy(np.ascontiguousarray(v)) for k, v in arrays.items()}, max_ctx=hb.max_ctx)
    dev = SimpleNamespace(arrays={k: v.to(device) for k, v in cpu.arrays.items()}, max_ctx=hb.max_ctx)
    return dev, cpu, n_pages


def close(got, want, dtype, what, f32=2e-5, bf16=2e-2):
    tol = bf16 if dtype == torch.bfloat16 else f32
    err = (got.double().cpu() - want.double().cpu()).abs().max().item() / max(want.double().abs().max().item(), 1e-30)
    assert err <= tol, f"{what}: relative error {err:.3e} over {tol:.1e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [40, 320, 1000, 4096])
def test_sandwich_norm(dtype, width):
    """Every form: a pre-norm alone, a branch normed, scaled and added with the next pre-norm in the same
    pass, the branch added as it is, no output, gathered rows (which leave the residual alone), the
    plain norm of rows that are no stream; centred and not, with and without biases."""
    o = ops()
    g = torch.Generator().manual_seed(width)
    n = 37
    res = torch.randn(n, width, generator=g) * 3 + 0.5
    br = (torch.randn(n, width, generator=g) * 2 - 0.3).to(dtype)
    mk = lambda: (torch.randn(width, generator=g) * 0.3 + 1).to(dtype)
    post, pre = (mk(), mk(), 1e-5, True), (mk(), mk(), 1e-6, True)
    rms = (mk(), None, 1e-5, False)
    rows = torch.tensor([5, 0, 36, 5], dtype=torch.int32)
    dev = lambda c: None if c is None else tuple(t.cuda() if torch.is_tensor(t) else t for t in c)
    cases = [(res, None, None, 1.0, pre, None), (res, br, post, 0.3, pre, None), (res, br, None, 1.0, pre, None),
             (res, br, post, 0.7, None, None), (res, br, post, 0.3, pre, rows), (res, None, None, 1.0, pre, rows),
             (None, br, None, 1.0, pre, None), (res, br, rms, 2.0, rms, None)]
    for i, (r, b, pa, scale, pb, idx) in enumerate(cases):
        r_ref = None if r is None else r.clone()
        want = R.sandwich_norm(r_ref, b, pa, scale, pb, idx, dtype)
        r_dev = None if r is None else r.clone().cuda()
        got = o.sandwich_norm(r_dev, None if b is None else b.cuda(), dev(pa), scale, dev(pb), None if idx is None else idx.cuda(), dtype)
        if pb is not None:
            close(got, want, dtype, f"case {i} output", bf16=1e-2)
        if r is not None:
            close(r_dev, r_ref, torch.float32, f"case {i} residual", f32=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_activation_and_scale(dtype):
    o = ops()
    x = (torch.randn(33, 77, generator=torch.Generator().manual_seed(1)) * 3).to(dtype)
    for kind in ("relu2", "silu", "gelu_tanh"):
        close(o.activation(x.cuda(), kind, dtype), R.activation(x, kind, dtype), dtype, kind, bf16=1e-2)
    y = torch.randn(5, 1001)
    close(o.scale_rows(y.clone().cuda(), 2.5), y * 2.5, torch.float32, "scale", f32=1e-7)


def rotation(rot_dim, positions, interleaved=True):
    ang = torch.outer(torch.arange(positions, dtype=torch.float32), 1.0 / (50.0 ** (torch.arange(0, rot_dim, 2).float() / rot_dim)))
    return Rotation((torch.cos(ang) * 1.1).contiguous(), (torch.sin(ang) * 1.1).contiguous(), rot_dim, interleaved)


def on_device(rot):
    return Rotation(rot.cos.cuda(), rot.sin.cuda(), rot.rotary_dim, rot.interleaved)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_rank,kv_rank,rot_dim", [(12, 20, 6), (128, 64, 16), (96, 512, 64), (9, 5, 2)])
def test_latent_prepare(dtype, q_rank, kv_rank, rot_dim):
    o = ops()
    page = 16
    dev, cpu, n_pages = context([(0, 21), (37, 1), (16, 2)], page)
    n = 24
    g = torch.Generator().manual_seed(q_rank)
    kv_col = q_rank + (-q_rank % 8)
    proj = (torch.randn(n, kv_col + kv_rank + rot_dim + 3, generator=g) * 2).to(dtype)
    qn, kn = (torch.randn(q_rank, generator=g) * 0.3 + 1).to(dtype), (torch.randn(kv_rank, generator=g) * 0.3 + 1).to(dtype)
    rot = rotation(rot_dim, 64)
    pages_ref = torch.zeros(n_pages, 1, page, kv_rank + rot_dim, dtype=dtype)
    pages_dev = pages_ref.clone().cuda()
    values_dev = torch.zeros(n_pages, 1, kv_rank, page, dtype=dtype).cuda()
    kw = dict(kv_col=kv_col, kv_rank=kv_rank, rot_dim=rot_dim, page_size=page)
    want = R.latent_prepare(proj, q_rank, qn, 1e-5, dtype, kv_norm=kn, rotation=rot, positions=cpu.arrays["positions"],
                            pages=pages_ref, slots=cpu.arrays["slots_g0"], **kw)
    got = o.latent_prepare(proj.cuda(), q_rank, qn.cuda(), 1e-5, dtype, kv_norm=kn.cuda(), rotation=on_device(rot),
                           positions=dev.arrays["positions"], pages=pages_dev, slots=dev.arrays["slots_g0"], values=values_dev, **kw)
    close(got, want, dtype, "query latent", bf16=1e-2)
    close(pages_dev, pages_ref, dtype, "page rows", bf16=1e-2)
    assert torch.equal(values_dev.transpose(2, 3), pages_dev[..., :kv_rank]), "the transposed copy holds the same latents"
    # a layer that reads another's cache writes nothing
    before = pages_dev.clone()
    o.latent_prepare(proj.cuda(), q_rank, qn.cuda(), 1e-5, dtype)
    assert torch.equal(before, pages_dev)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,in_dim,out_dim,tail", [(3, 10, 20, 6), (8, 32, 64, 16), (2, 128, 512, 64), (5, 7, 300, 0)])
def test_head_linear(dtype, heads, in_dim, out_dim, tail):
    """Into the latent's space (a turned tail behind every head's product, float32 out) and out of it
    (float32 in, a sigmoid gate per head, the activation dtype out)."""
    o = ops()
    n = 19
    g = torch.Generator().manual_seed(heads)
    x = torch.randn(n, heads * (in_dim + tail), generator=g).to(dtype)
    w = (torch.randn(heads, in_dim, out_dim, generator=g) / in_dim ** 0.5).to(dtype)
    pos = torch.randint(0, 64, (n,), generator=g, dtype=torch.int32)
    rot = rotation(tail, 64) if tail else None
    want = R.head_linear(x, w, heads, in_dim, out_dim, torch.float32, tail=tail, rotation=rot, positions=pos)
    got = o.head_linear(x.cuda(), w.cuda(), heads, in_dim, out_dim, torch.float32, tail=tail, rotation=on_device(rot) if tail else None,
                        positions=pos.cuda())
    close(got, want, torch.float32, "into the latent", f32=2e-5)
    xo = torch.randn(n, heads * in_dim, generator=g)
    gate = torch.randn(n, heads + 11, generator=g).to(dtype)
    want = R.head_linear(xo, w, heads, in_dim, out_dim, dtype, gate=gate, gate_col=7)
    got = o.head_linear(xo.cuda(), w.cuda(), heads, in_dim, out_dim, dtype, gate=gate.cuda(), gate_col=7)
    close(got, want, dtype, "out of the latent", bf16=1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_rank,rot_dim", [(2, 64, 16), (5, 20, 6), (16, 512, 64), (1, 130, 2)])
@pytest.mark.parametrize("special", [0, 15, 16, 63, 64, 127, 128, 3, 399, 400])
def test_one_row_stands_out_at_every_border(dtype, heads, kv_rank, rot_dim, special):
    """Page rows of 700 tokens, one of which scores far above the rest and carries a latent unlike any
    other; a prompt's portion at positions 380..449 (row 399 is inside for some of its tokens, row 400
    for fewer, both cut by the portion's own causal edge), single tokens at 399, 400, 699 and 16: rows 15 /
    16, 63 / 64 and 127 / 128 lie across borders of pages and of the blocks of keys the kernel stages."""
    if heads == 16 and special not in (0, 63, 64, 400):
        pytest.skip("the largest size runs a few of the borders")
    o = ops()
    page, L = 16, 700
    width = kv_rank + rot_dim
    g = torch.Generator().manual_seed(special + heads)
    rows = torch.randn(L, width, generator=g) * 0.2
    rows[special, 0] = 30.0
    rows = rows.to(dtype).float()
    spans_at = [(380, 70), (399, 1), (400, 1), (699, 1), (16, 1)]
    tile = o.latent_tile_tokens(heads)
    dev, cpu, n_pages = context(spans_at, page, tile_tokens=tile)
    pages = torch.zeros(n_pages, 1, page, width)
    bt = cpu.arrays["block_table_g0"]
    for s, (p0, n) in enumerate(spans_at):
        for j in range(p0 + n):
            pages[int(bt[s, j // page]), 0, j % page] = rows[j]
    pages = pages.to(dtype)
    n_tok = sum(n for _, n in spans_at)
    q = torch.randn(n_tok, heads, width, generator=g) * 0.3
    q[:, :, 0] = 1.0
    scale = 0.7
    got = o.latent_attention(q.reshape(n_tok, -1).cuda(), pages.cuda(), heads, kv_rank, rot_dim, scale, dev, 0, page,
                             tiles=dev.arrays[f"latent_tiles_{tile}"])
    pos = cpu.arrays["positions"]
    want = torch.empty(n_tok, heads, kv_rank, dtype=torch.float64)
    for t in range(n_tok):
        keys = rows[: int(pos[t]) + 1].double()
        want[t] = torch.softmax(q[t].double() @ keys.T * scale, dim=-1) @ keys[:, :kv_rank]
    close(got, want.reshape(n_tok, -1), torch.float32, f"row {special}", f32=2e-5)
    seen = [t for t in range(n_tok) if int(pos[t]) >= special]
    if seen:  # where the row is visible it carries nearly all the weight: its own latent comes back
        assert (got[seen].view(len(seen), heads, kv_rank)[:, :, 0].cpu() > 20.0).all()


@pytest.mark.parametrize("heads,in_dim,out_dim,tail,n", [(3, 32, 48, 8, 40), (16, 128, 512, 64, 150), (5, 512, 128, 0, 77), (2, 64, 16, 16, 33)])
def test_head_linear_on_matrix_cores(heads, in_dim, out_dim, tail, n):
    """Many tokens, bfloat16 weights kept transposed: into the latent (bfloat16 in, a turned tail, float32
    out) and out of it (float32 in as two bfloat16 parts, gates, bfloat16 out; also float32 out of the same
    input to see that nothing of it was rounded away); token tiles that end
    inside a wave's 16 rows, column tiles that end inside a workgroup's 64."""
    o = ops()
    g = torch.Generator().manual_seed(n)
    bf = torch.bfloat16
    w = (torch.randn(heads, in_dim, out_dim, generator=g) / in_dim ** 0.5).to(bf)
    w_t = o.head_weights_transposed(w.cuda())
    assert w_t is not None and tuple(w_t.shape) == (heads, out_dim, in_dim)
    pos = torch.randint(0, 64, (n,), generator=g, dtype=torch.int32)
    rot = rotation(tail, 64) if tail else None
    x = torch.randn(n, heads * (in_dim + tail), generator=g).to(bf)
    want = R.head_linear(x, w, heads, in_dim, out_dim, torch.float32, tail=tail, rotation=rot, positions=pos)
    got = o.head_linear(x.cuda(), w.cuda(), heads, in_dim, out_dim, torch.float32, tail=tail, rotation=on_device(rot) if tail else None,
                        positions=pos.cuda(), w_t=w_t)
    close(got, want, torch.float32, "into the latent", f32=2e-5)
    xo = torch.randn(n, heads * in_dim, generator=g)  # (float32 values bfloat16 does not hold: they go in as two parts)
    gate = torch.randn(n, heads + 11, generator=g).to(bf)
    want = R.head_linear(xo, w, heads, in_dim, out_dim, bf, gate=gate, gate_col=7)
    got = o.head_linear(xo.cuda(), w.cuda(), heads, in_dim, out_dim, bf, gate=gate.cuda(), gate_col=7, w_t=w_t)
    close(got, want, bf, "out of the latent", bf16=1e-2)
    # the same sums before their rounding: against the plain float32 product they differ by 2^-16 of the input, not 2^-8
    exact = R.head_linear(xo, w, heads, in_dim, out_dim, torch.float32, gate=gate, gate_col=7)
    assert (got.float().cpu() - exact.to(bf).float()).abs().max() <= 2.0 ** -7 * exact.abs().max()


@pytest.mark.parametrize("heads,kv_rank,rot_dim,page", [(2, 64, 32, 32), (5, 128, 32, 64), (16, 512, 64, 64), (20, 256, 64, 32)])
@pytest.mark.parametrize("special", [0, 31, 32, 63, 64, 399, 400])
@pytest.mark.parametrize("splits", [1, 3, None])
def test_matrix_core_form_at_every_border(heads, kv_rank, rot_dim, page, special, splits):
    """The same towering row for the matrix-core form (bfloat16 pages, the latent a second time in
    transposed pages): borders of its groups of 32 keys and of pages, tiles of several tokens where
    heads are few and of one token's heads in chunks of 16 where they are many, the keys whole,
    divided in three, and divided as the library decides; against float64 over the same rounded rows."""
    if kv_rank >= 256 and special not in (0, 63, 64, 400):
        pytest.skip("the largest sizes run a few of the borders")
    o = ops()
    assert o.latent_attention_on_matrix_cores(torch.bfloat16, kv_rank, rot_dim, page)
    L, width = 700, kv_rank + rot_dim
    g = torch.Generator().manual_seed(special + heads)
    rows = torch.randn(L, width, generator=g) * 0.2
    rows[special, 0] = 30.0
    rows = rows.to(torch.bfloat16).float()
    spans_at = [(380, 70), (399, 1), (400, 1), (699, 1), (16, 1)]
    tile = o.latent_tile_tokens(heads, True)
    dev, cpu, n_pages = context(spans_at, page, tile_tokens=tile)
    pages = torch.full((n_pages, 1, page, width), 7.0)  # (slots never written hold something)
    bt = cpu.arrays["block_table_g0"]
    for s, (p0, n) in enumerate(spans_at):
        for j in range(p0 + n):
            pages[int(bt[s, j // page]), 0, j % page] = rows[j]
    values = pages[..., :kv_rank].transpose(2, 3).contiguous()
    n_tok = sum(n for _, n in spans_at)
    q = (torch.randn(n_tok, heads, width, generator=g) * 0.3)
    q[:, :, 0] = 1.0
    q = q.to(torch.bfloat16).float()  # what the kernel rounds its queries to
    scale = 0.7
    got = o.latent_attention(q.reshape(n_tok, -1).cuda(), pages.to(torch.bfloat16).cuda(), heads, kv_rank, rot_dim, scale, dev, 0, page,
                             tiles=dev.arrays[f"latent_tiles_{tile}"], values=values.to(torch.bfloat16).cuda(), splits=splits)
    pos = cpu.arrays["positions"]
    want = torch.empty(n_tok, heads, kv_rank, dtype=torch.float64)
    for t in range(n_tok):
        keys = rows[: int(pos[t]) + 1].double()
        want[t] = torch.softmax(q[t].double() @ keys.T * scale, dim=-1) @ keys[:, :kv_rank]
    close(got, want.reshape(n_tok, -1), torch.bfloat16, f"row {special}", bf16=1e-2)
    seen = [t for t in range(n_tok) if int(pos[t]) >= special]
    if seen:
        assert (got[seen].view(len(seen), heads, kv_rank)[:, :, 0].cpu() > 20.0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 4, 5])
def test_convolution_with_silu_and_its_state(dtype, taps):
    """Spans shorter and longer than the taps, behind states that hold earlier inputs; then the state
    takes the span in (a span of one token shifts it by one)."""
    o = ops()
    channels = 52
    spans_at = [(0, 9), (30, 1), (7, 2), (12, taps + 3)]
    dev, cpu, _ = context(spans_at, 16, slots=[2, 0, 3, 1])
    n = sum(k for _, k in spans_at)
    g = torch.Generator().manual_seed(taps)
    x = torch.randn(n, channels + 4, generator=g).to(dtype)[:, :channels]  # a view with a row stride
    w = (torch.randn(channels, taps, generator=g) * 0.5).to(dtype)
    state = torch.randn(4, max(taps - 1, 1), channels, generator=g).to(dtype)[:, : taps - 1]
    state = state.contiguous()
    want = R.causal_conv_act(x, w, None, state, cpu, act="silu")
    xd = x.cuda()
    sd = state.clone().cuda()
    got = o.causal_conv(xd, w.cuda(), None, sd if taps > 1 else None, dev, act="silu")
    close(got, want, dtype, "convolution", bf16=1e-2)
    if taps > 1:
        R.conv_state_push(x, state, cpu)
        o.conv_state_push(xd, sd, dev)
        assert torch.equal(sd.cpu(), state)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["delta", "gla"])
@pytest.mark.parametrize("heads,kv,dim,vdim", [(4, 2, 12, 10), (2, 2, 24, 9), (2, 2, 64, 32), (3, 1, 128, 70), (1, 1, 200, 5), (2, 1, 16, 300), (1, 1, 300, 40), (2, 1, 8, 20), (1, 1, 600, 6)])
def test_linear_state_scan(dtype, kind, heads, kv, dim, vdim):
    """Both kinds of write and of decay, key channels from fewer than a lane's share to many lanes a
    column, more value columns than a workgroup holds; spans of one token and of several staged chunks,
    behind states that are not zero; and a span cut in two gives the same state and outputs bit for bit."""
    o = ops()
    if kind == "gla":
        kv = heads
    spans_at = [(0, 37), (5, 1), (9, 18)]
    dev, cpu, _ = context(spans_at, 16, slots=[1, 3, 0])
    n = sum(k for _, k in spans_at)
    g = torch.Generator().manual_seed(dim + vdim)
    qkv = torch.randn(n, 2 * kv * dim + heads * vdim + 5, generator=g).to(dtype)
    state = torch.randn(4, heads, dim, vdim, generator=g) * 0.5
    if kind == "delta":
        ba = torch.randn(n, 2 * heads + 3, generator=g)
        a_log, dt = torch.randn(heads, generator=g) * 0.5, torch.randn(heads, generator=g) * 0.5
        args = lambda f: dict(q_scale=dim ** -0.5, unit_eps=1e-6, decay=("head", f(ba), heads + 1, f(a_log), f(dt)), beta=(f(ba), 1))
    else:
        z = torch.randn(n, heads * dim + 2, generator=g) * 2
        bias = torch.randn(heads * dim, generator=g)
        args = lambda f: dict(q_scale=dim ** -0.5, unit_eps=None, decay=("channel", f(z), 2, f(bias), 3.5), beta=None)
    s_ref = state.clone()
    want = R.linear_state_scan(qkv, heads, kv, dim, vdim, s_ref, cpu, **args(lambda t: t))
    s_dev = state.clone().cuda()
    got = o.linear_state_scan(qkv.cuda(), heads, kv, dim, vdim, s_dev, dev, **args(lambda t: t.cuda()))
    close(got, want, torch.float32, "read-outs", f32=5e-5)
    close(s_dev, s_ref, torch.float32, "states", f32=5e-5)
    # the first request's span in two steps (20 + 17 tokens): the same bits
    s_two = state.clone().cuda()
    outs = []
    for p0, cnt, lo in ((0, 20, 0), (20, 17, 20)):
        d2, _, _ = context([(p0, cnt)], 16, slots=[1])
        part = lambda t, lo=lo, cnt=cnt: t[lo: lo + cnt].contiguous().cuda() if t.dim() == 2 and t.shape[0] == n else t.cuda()
        outs.append(o.linear_state_scan(part(qkv), heads, kv, dim, vdim, s_two, d2, **args(part)))
    assert torch.equal(torch.cat(outs), got[:37]) and torch.equal(s_two[1], s_dev[1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,vdim", [(4, 10), (2, 64), (3, 200)])
def test_gated_head_norm(dtype, heads, vdim):
    o = ops()
    g = torch.Generator().manual_seed(vdim)
    n = 21
    x = torch.randn(n, heads * vdim, generator=g) * 4
    w = (torch.randn(vdim, generator=g) * 0.3 + 1).to(dtype)
    gate = torch.randn(n, heads * vdim + 9, generator=g).to(dtype)
    want = R.gated_head_norm(x, w, 1e-5, gate, 9, heads, vdim, dtype)
    got = o.gated_head_norm(x.cuda(), w.cuda(), 1e-5, gate.cuda(), 9, heads, vdim, dtype)
    close(got, want, dtype, "head norm", bf16=1e-2)
