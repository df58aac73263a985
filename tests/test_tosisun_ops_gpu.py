"""The kernels behind the Tosisun design, each alone against the plain implementation's function of the same
mechanism: the layer norm in its forms, the convolved and normed projections with their tail, attention with a sink
through every attention kernel (keys far away, at the borders of pages, chunks and cuts), the router, the
activations, the soft cap."""
import math

import numpy as np
import pytest
import torch

from plain import tosisun_plain as plain
from zedinfer_amd import ops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _close(got, want, tol, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    scale = max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= tol * scale, (what, err, scale)


# ---- layer norm -----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n, H", [(1, 40), (3, 96), (70, 200), (130, 1024), (5, 4100), (66, 1100), (2, 50), (70, 1030), (5, 4098),
                                  (3, 8200)])
def test_layer_norm_alone_and_on_a_sublayers_output(n, H):
    g = torch.Generator().manual_seed(n * 1000 + H)
    x = torch.randn(n, H, generator=g) * 3 + 0.7
    w, b = 1 + 0.2 * torch.randn(H, generator=g), 0.3 * torch.randn(H, generator=g)
    want = plain.layer_norm(x.double(), w.double(), b.double(), 1e-5)
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    _close(ops.layer_norm(xd, wd, bd, 1e-5), want, 2e-6, "alone")
    # a constant row: zero deviations, the bias alone is left
    flat = torch.full((n, H), 2.5, device=DEV)
    _close(ops.layer_norm(flat, wd, bd, 1e-5), b.double().expand(n, H), 1e-6, "flat")
    # on an output: the stream takes the normed rows, the copy is the new stream
    resid = torch.randn(n, H, generator=g)
    rd = resid.to(DEV)
    copy = torch.empty(n, H, dtype=torch.bfloat16, device=DEV)
    ops.layer_norm(xd, wd, bd, 1e-5, out=copy, resid=rd)
    _close(rd, resid.double() + want, 2e-6, "stream")
    assert torch.equal(copy, rd.to(torch.bfloat16))
    # a stack of terms is added first; bfloat16 rows are read as they are
    parts = torch.randn(3, n, H, generator=g)
    rd2 = resid.to(DEV)
    ops.layer_norm(parts.to(DEV), wd, bd, 1e-5, resid=rd2)
    _close(rd2, resid.double() + plain.layer_norm(parts.double().sum(0), w.double(), b.double(), 1e-5), 3e-6, "stack")
    xb = x.to(torch.bfloat16)
    _close(ops.layer_norm(xb.to(DEV), wd, bd, 1e-5, out_dtype=torch.float32),
           plain.layer_norm(xb.double(), w.double(), b.double(), 1e-5), 2e-6, "bf16 rows")


# ---- the convolved, normed and turned projections ----------------------------------------------------------------
def _paged(n_tokens, ps, seed, spare=3):
    """A block table that scatters the pages of one sequence over a pool, and every token's slot."""
    pages = -(-n_tokens // ps)
    perm = torch.randperm(pages + spare, generator=torch.Generator().manual_seed(seed))[:pages]
    table = perm.to(torch.int32)
    pos = torch.arange(n_tokens)
    slots = (table[pos // ps].long() * ps + pos % ps).to(torch.int32)
    return table.view(1, -1), slots, pages + spare


@pytest.mark.parametrize("nh, nkv, dim, vdim, D, taps, rot, dtype", [
    (6, 2, 32, 16, 32, 4, 8, torch.float32), (4, 4, 16, 48, 48, 2, 16, torch.bfloat16), (3, 1, 24, 24, 32, 1, 0, torch.bfloat16),
    (2, 1, 8, 72, 80, 5, 4, torch.bfloat16), (5, 5, 20, 12, 20, 3, 20, torch.float32)])
def test_conv_qkv_in_portions_is_the_whole_sequences(nh, nkv, dim, vdim, D, taps, rot, dtype):
    T, ps = 37, 8
    g = torch.Generator().manual_seed(nh * 100 + taps)
    Qd, Kd, Vd = nh * dim, nkv * dim, nkv * vdim
    C = Qd + Kd + Vd
    proj = torch.randn(T, C, generator=g)
    bias = 0.5 * torch.randn(C, generator=g)
    conv_w = 0.6 * torch.randn(C, taps, generator=g)
    qn, kn = 1 + 0.2 * torch.randn(Qd, generator=g), 1 + 0.2 * torch.randn(Kd, generator=g)
    freqs = plain.stretched_frequencies(rot, 100.0, None) if rot else []
    # the plain way
    y = plain.short_conv(proj.double() + bias.double(), conv_w.double())
    q = plain.rms(y[:, :Qd], 1e-5) * qn.double()
    k = plain.rms(y[:, Qd:Qd + Kd], 1e-5) * kn.double()
    pos = torch.arange(T)
    q = plain.rotate_half(q.view(T, nh, dim), pos, freqs) if rot else q.view(T, nh, dim)
    k = plain.rotate_half(k.view(T, nkv, dim), pos, freqs) if rot else k.view(T, nkv, dim)
    v = y[:, Qd + Kd:].view(T, nkv, vdim)
    # the kernels, in portions (one shorter than the tail), in the second of three state slots
    table, slots, pages = _paged(T, ps, seed=taps)
    kc = torch.full((pages, nkv, ps, D), 7.0, dtype=dtype, device=DEV)
    vc = torch.full((pages, nkv, D, ps), 7.0, dtype=dtype, device=DEV)
    state = torch.zeros(3, ops.conv_state_floats(C, taps), device=DEV)
    state[0] = 9.0
    state[2] = -9.0
    q_all = torch.empty(T, nh * D, dtype=dtype, device=DEV)
    inv = torch.tensor(freqs, dtype=torch.float32, device=DEV)
    at = 0
    for n in (1, 2, 9, 1, 3, 2, 19):
        posd = torch.arange(at, at + n, dtype=torch.int32, device=DEV)
        tab = ops.rope_table(posd, inv) if rot else None
        qo = torch.empty(n, nh * D, dtype=dtype, device=DEV)
        pr = proj[at:at + n].to(DEV)
        es, el, sl = (torch.tensor([x], dtype=torch.int32, device=DEV) for x in (0, n, 1))
        ops.conv_qkv(pr, bias.to(DEV), conv_w.to(DEV), state, qn.to(DEV), kn.to(DEV), 1e-5, tab,
                     torch.zeros(n, dtype=torch.int32, device=DEV), es, sl, slots[at:at + n].to(DEV), kc, vc, nh, nkv, dim, vdim,
                     D, taps, qo)
        ops.conv_tail(state, pr, bias.to(DEV), es, el, sl, taps)
        q_all[at:at + n] = qo
        at += n
    assert at == T
    tol = 3e-6 if dtype == torch.float32 else 1e-2
    qg = q_all.view(T, nh, D)
    _close(qg[:, :, :dim], q, tol, "q")
    assert float(qg[:, :, dim:].abs().max()) == 0.0 if D > dim else True
    pg = (slots // ps).long()
    kg = kc[pg, :, (slots % ps).long(), :]            # [T, nkv, D]
    vg = vc[pg, :, :, (slots % ps).long()]            # [T, nkv, D]
    _close(kg[:, :, :dim], k, tol, "k")
    _close(vg[:, :, :vdim], v, tol, "v")
    if D > dim:
        assert float(kg[:, :, dim:].abs().max()) == 0.0
    if D > vdim:
        assert float(vg[:, :, vdim:].abs().max()) == 0.0
    # the other requests' tails were left alone, and this one holds the last rows that entered the convolution
    assert float((state[0] - 9.0).abs().max()) == 0.0 and float((state[2] + 9.0).abs().max()) == 0.0
    if taps > 1:
        _close(state[1, :(taps - 1) * C].view(taps - 1, C), (proj + bias)[T - (taps - 1):], 1e-6, "tail")
        # tokens without a place in the cache stand behind an entry's own and do not move the tail; an entry that has
        # none of its own (it names slot 0) leaves that slot's tail alone
        before = state.clone()
        pr = torch.randn(7, C, generator=g).to(DEV)
        i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)      # noqa: E731
        ops.conv_tail(state, pr, bias.to(DEV), i32([0, 5]), i32([5, 2]), i32([1, 0]), taps, slots=i32([3, 4, -1, -1, -1, -1, -1]))
        assert torch.equal(state[0], before[0]) and torch.equal(state[2], before[2])
        rows = torch.cat([before[1, :(taps - 1) * C].view(taps - 1, C), pr[:2] + bias.to(DEV)])[-(taps - 1):]
        _close(state[1, :(taps - 1) * C].view(taps - 1, C), rows, 1e-6, "tail under padding")


# ---- attention with a sink ---------------------------------------------------------------------------------------
def _attention_case(T, nh, nkv, d, ps, seed, far=None):
    """Random queries, keys and values of one sequence in scattered pages; with ``far`` = (query position, key
    position) that query's key is scaled so that its score stands out among all the others."""
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(T, h, d, generator=g) for h in (nh, nkv, nkv))
    if far is not None:
        qp, kp = far
        for h in range(nh):
            k[kp, h // (nh // nkv)] = 0
        for gg in range(nkv):
            k[kp, gg] = q[qp, gg * (nh // nkv)] * 4.0          # the first head of every group looks straight at it
    return q, k, v


def _fill_cache(k, v, ps, seed, dtype):
    T, nkv, d = k.shape
    table, slots, pages = _paged(T, ps, seed)
    kc = torch.zeros(pages, nkv, ps, d, dtype=dtype)
    vc = torch.zeros(pages, nkv, d, ps, dtype=dtype)
    pg, off = (slots // ps).long(), (slots % ps).long()
    kc[pg, :, off, :] = k.to(dtype)
    vc[pg, :, :, off] = v.to(dtype)
    return table.to(DEV), kc.to(DEV), vc.to(DEV)


@pytest.mark.parametrize("T, nh, nkv, d, ps", [(1, 2, 1, 16, 8), (70, 6, 2, 32, 8), (300, 4, 4, 48, 16), (530, 3, 1, 24, 4),
                                               (90, 20, 1, 16, 8), (40, 1, 1, 144, 8)])
def test_the_plain_kernel_counts_the_sink_once(T, nh, nkv, d, ps):
    q, k, v = _attention_case(T, nh, nkv, d, ps, seed=T, far=(T - 1, T // 3) if T > 3 else None)
    sink = 1.5 * torch.randn(nh, generator=torch.Generator().manual_seed(1))
    scale = 1.0 / math.sqrt(d)
    want = plain.sink_attention(q.double(), k.double(), v.double(), scale, sink.double(), nh // nkv)
    table, kc, vc = _fill_cache(k, v, ps, seed=T, dtype=torch.float32)
    tok_seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    pos = torch.arange(T, dtype=torch.int32, device=DEV)
    got = ops.attention(q.reshape(T, nh * d).to(DEV), kc, vc, tok_seq, pos, table, nh, nkv, d, scale, sinks=sink.to(DEV))
    _close(got.view(T, nh, d), want, 5e-6, "sink")
    # no sink at all is a sink of minus infinity, and differs from a sink of zero
    none = ops.attention(q.reshape(T, nh * d).to(DEV), kc, vc, tok_seq, pos, table, nh, nkv, d, scale)
    want_none = plain.sink_attention(q.double(), k.double(), v.double(), scale, torch.full((nh,), -1e30, dtype=torch.float64), nh // nkv)
    _close(none.view(T, nh, d), want_none, 5e-6, "no sink")
    assert float((none - got).abs().max()) > 1e-3


@pytest.mark.parametrize("T, nh, nkv, d, ps, far", [
    (255, 4, 2, 64, 16, (254, 0)), (256, 4, 2, 64, 16, (255, 1)), (257, 8, 2, 64, 16, (256, 0)), (513, 6, 2, 32, 8, (512, 255)),
    (1300, 4, 4, 48, 16, (1299, 256)), (2100, 2, 1, 128, 32, (2099, 3)), (700, 16, 1, 16, 64, (699, 300)),
    (97, 3, 1, 80, 8, (96, 15)), (1, 2, 1, 16, 8, None)])
def test_decoded_tokens_over_chunks_of_keys_count_the_sink_once(T, nh, nkv, d, ps, far):
    """The last tokens of a sequence, one query each, through the kernel that cuts a query's keys into chunks of 256
    and merges them: a key far back, in the first chunk or just across a chunk's border, must carry its weight, and
    the sink must count once, not once a chunk."""
    q, k, v = _attention_case(T, nh, nkv, d, ps, seed=T + 1, far=far)
    q, k, v = (x.to(torch.bfloat16) for x in (q, k, v))
    sink = torch.tensor([(-1) ** h * (0.5 + h) for h in range(nh)], dtype=torch.float32)
    scale = 1.0 / math.sqrt(d)
    want = plain.sink_attention(q.double(), k.double(), v.double(), scale, sink.double(), nh // nkv)
    if far is not None:                    # the far key does carry the weight in the plain result
        h0 = 0
        w_far = torch.softmax(torch.cat([(k[:far[0] + 1, 0].double() @ q[far[0], h0].double()) * scale, sink[h0:h0 + 1].double()]), 0)
        assert float(w_far[far[1]]) > 0.9
    assert ops.attention_decode_supported(torch.bfloat16, nh, nkv, d, ps)
    table, kc, vc = _fill_cache(k, v, ps, seed=T, dtype=torch.bfloat16)
    last = list(range(max(0, T - 3), T))
    idx = torch.tensor(last, dtype=torch.int32, device=DEV)
    tok_seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    pos = torch.arange(T, dtype=torch.int32, device=DEV)
    out = torch.zeros(T, nh * d, dtype=torch.bfloat16, device=DEV)
    ops.attention_decode(q.reshape(T, nh * d).to(DEV), kc, vc, tok_seq, pos, table, nh, nkv, d, scale, T, out=out,
                         tok_index=idx, sinks=sink.to(DEV))
    _close(out.view(T, nh, d)[last], want[last], 1.2e-2, "decode")


@pytest.mark.parametrize("T, past, nh, nkv, d, ps, far", [
    (130, 0, 4, 2, 64, 16, (129, 0)), (70, 500, 6, 2, 32, 8, (569, 7)), (2300, 0, 2, 1, 64, 16, (2299, 1)),
    (300, 2040, 2, 2, 128, 16, (2339, 2047)), (300, 2040, 2, 2, 128, 16, (2339, 2048)), (200, 1990, 3, 1, 48, 32, (2100, 40)),
    (5, 3, 2, 1, 16, 8, None)])
def test_portions_of_prompts_over_cuts_of_keys_count_the_sink_once(T, past, nh, nkv, d, ps, far):
    """A portion of T tokens after ``past`` cached ones through the matrix-core prompt kernel: tiles that see more
    than 2,048 keys are cut over several workgroups and merged, and the sink must count once."""
    total = past + T
    q, k, v = _attention_case(total, nh, nkv, d, ps, seed=total, far=far)
    q, k, v = (x.to(torch.bfloat16) for x in (q, k, v))
    sink = torch.tensor([1.0 - 0.7 * h for h in range(nh)], dtype=torch.float32)
    scale = 1.0 / math.sqrt(d)
    rows = list(range(past, total, 7)) + [total - 1] + ([far[0]] if far else [])
    want = plain.sink_attention(q.double(), k.double(), v.double(), scale, sink.double(), nh // nkv)
    assert ops.attention_prefill_supported(torch.bfloat16, nh, nkv, d, ps)
    table, kc, vc = _fill_cache(k, v, ps, seed=T, dtype=torch.bfloat16)
    tile = ops.attention_prefill_tile_min()
    offs = list(range(0, T, tile))
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)      # noqa: E731
    out = torch.zeros(T, nh * d, dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(q[past:].reshape(T, nh * d).to(DEV), kc, vc, i32([0] * len(offs)), i32(offs), i32([0]), i32([T]),
                          i32([past]), table, nh, nkv, d, scale, out=out, max_keys=total, sinks=sink.to(DEV))
    _close(out.view(T, nh, d)[[r - past for r in rows]], want[rows], 1.2e-2, "prefill")


# ---- router, activations, cap -------------------------------------------------------------------------------------
@pytest.mark.parametrize("n, E, top", [(1, 2, 1), (7, 6, 3), (33, 16, 2), (5, 70, 6), (9, 300, 300), (4, 5, 5)])
def test_the_router_of_largest_logits(n, E, top):
    g = torch.Generator().manual_seed(E)
    z = torch.randn(n, E, generator=g)
    z[0, : min(E, 4)] = 1.25                          # equals: the lower index first
    bias = torch.randn(E, generator=g)
    bias[: min(E, 4)] = 0.5
    idx = torch.empty(n, top, dtype=torch.int32, device=DEV)
    wt = torch.empty(n, top, dtype=torch.float32, device=DEV)
    ops.moe_route_top(z.to(DEV), bias.to(DEV), top, idx, wt)
    want_idx, want_wt = plain.route((z + bias).double(), top)
    assert idx.cpu().tolist() == want_idx.tolist()
    _close(wt, want_wt, 2e-6, "weights")
    assert torch.allclose(wt.sum(1).cpu(), torch.ones(n), atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_activations_and_cap(dtype):
    g = torch.Generator().manual_seed(5)
    n, I = 19, 52
    gu = (3 * torch.randn(n, 2 * I + 4, generator=g)).to(dtype)
    gate, up = gu[:, :I], gu[:, I + 4:]
    out = torch.empty(n, I, dtype=torch.float32, device=DEV)
    gd = gu.to(DEV)
    ops.clamped_glu(gd[:, :I], gd[:, I + 4:], 1.5, out=out)
    gg = torch.clamp(gate.double(), max=1.5)
    uu = torch.clamp(up.double(), -1.5, 1.5)
    _close(out, gg * torch.sigmoid(1.702 * gg) * (uu + 1), 2e-6, "clamped")
    assert float(out.max()) <= 1.5 * 2.5 + 1e-5
    z = (2 * torch.randn(n, I, generator=g)).to(dtype)
    o2 = torch.empty(n, I, dtype=torch.float32, device=DEV)
    ops.relu_squared(z.to(DEV), out=o2)
    _close(o2, torch.clamp(z.double(), min=0) ** 2, 2e-6, "relu squared")
    if dtype == torch.float32:
        parts = torch.randn(3, n, I, generator=g)
        ops.relu_squared(parts.to(DEV), out=o2)
        _close(o2, torch.clamp(parts.double().sum(0), min=0) ** 2, 3e-6, "relu squared of sums")
        x = 40 * torch.randn(n, I, generator=g)
        xd = x.to(DEV)
        ops.softcap(xd, 12.0)
        _close(xd, 12.0 * torch.tanh(x.double() / 12.0), 2e-6, "cap")
        assert float(xd.abs().max()) <= 12.0


@pytest.mark.parametrize("T, n, nh, nkv, d, ps", [(300, 3, 4, 2, 64, 16), (1100, 8, 12, 2, 128, 16), (40, 16, 6, 6, 32, 8), (257, 1, 20, 4, 48, 8)])
def test_the_projection_that_merges_the_chunks_counts_the_sink_once(T, n, nh, nkv, d, ps):
    """Decoded tokens of n sequences (here: the same keys at n lengths): the attention kernel leaves the chunks of
    keys unmerged, the output projection merges them; against the plain attention and a plain product."""
    g = torch.Generator().manual_seed(T)
    q, k, v = _attention_case(T, nh, nkv, d, ps, seed=T + 5, far=(T - 1, 2))
    q, k, v = (x.to(torch.bfloat16) for x in (q, k, v))
    sink = torch.tensor([2.0 - 0.9 * h for h in range(nh)], dtype=torch.float32)
    w = (torch.randn(72, nh * d, generator=g) / (nh * d) ** 0.5).to(torch.bfloat16)
    scale = 1.0 / math.sqrt(d)
    att = plain.sink_attention(q.double(), k.double(), v.double(), scale, sink.double(), nh // nkv)
    table, kc, vc = _fill_cache(k, v, ps, seed=T, dtype=torch.bfloat16)
    # sequence i holds the first T - i tokens: its decoded token is the one at position T - 1 - i
    pos = torch.tensor([T - 1 - i for i in range(n)], dtype=torch.int32, device=DEV)
    qs = torch.stack([q[T - 1 - i].reshape(nh * d) for i in range(n)]).to(DEV)
    tables = table.expand(n, -1).contiguous()
    tok_seq = torch.arange(n, dtype=torch.int32, device=DEV)
    assert ops.attention_decode_project_supported(w.to(DEV), n, nh, d)
    ws = torch.empty(ops.attention_decode_workspace(n, nh, d), dtype=torch.float32, device=DEV)
    assert ops.attention_decode(qs, kc, vc, tok_seq, pos, tables, nh, nkv, d, scale, T, workspace=ws, sinks=sink.to(DEV),
                                leave_chunks=True) is None
    sums = ops.attention_decode_project(ws, w.to(DEV), pos, nh, d, T, sinks=sink.to(DEV))
    want = torch.stack([att[T - 1 - i].reshape(nh * d) for i in range(n)]) @ w.double().T
    _close(sums.sum(0), want, 1.5e-2, "merged in the projection")
    # without the sink the same call gives another result (the first heads' sinks are of the size of the scores)
    other = ops.attention_decode_project(ws, w.to(DEV), pos, nh, d, T)
    assert float((other.sum(0) - sums.sum(0)).abs().max()) > 1e-4


# ---- the feed-forwards as parts --------------------------------------------------------------------------------------
def _part(registry, kind, params, weights, dtype):
    from zedinfer_amd.config.forward_config import PartSpec
    from zedinfer_amd.parts import Runtime
    rt = Runtime(DEV, dtype)
    spec = PartSpec(kind, params, {k: k for k in weights})
    return registry.get(kind)(spec, {k: v.to(DEV, dtype) for k, v in weights.items()}, rt)


def _sum_terms(y):
    return (y.sum(0) if y.dim() == 3 else y).double().cpu()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n, H, I", [(1, 64, 40), (9, 96, 136), (70, 72, 52), (200, 128, 256)])
def test_the_relu_squared_feed_forward(n, H, I, dtype):
    from zedinfer_amd.parts import FEED_FORWARDS
    g = torch.Generator().manual_seed(n + I)
    w = {"up": torch.randn(I, H, generator=g) / H ** 0.5, "down": torch.randn(H, I, generator=g) / I ** 0.5}
    w = {k: v.to(dtype) for k, v in w.items()}
    x = torch.randn(n, H, generator=g).to(dtype)
    ff = _part(FEED_FORWARDS, "relu2_mlp", {"hidden_size": H, "intermediate_size": I}, w, dtype)
    got = _sum_terms(ff.forward(x.to(DEV)))
    want = plain.relu_squared_mlp(x.double(), w["up"].double(), w["down"].double())
    _close(got, want, 1e-5 if dtype == torch.float32 else 2e-2, "relu squared mlp")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n, H, E, top, ff, sff", [(1, 64, 4, 2, 24, 16), (13, 96, 6, 3, 40, 56), (90, 72, 5, 1, 36, 0),
                                                 (300, 128, 16, 4, 64, 96), (7, 48, 3, 3, 20, 12)])
def test_the_clamped_experts(n, H, E, top, ff, sff, dtype):
    """Router with bias, the choice of the largest logits, clamped experts, the shared expert: against the plain
    feed-forward.  The tokens' router logits are spread so that no choice is a close call under rounding."""
    from zedinfer_amd.parts import FEED_FORWARDS
    g = torch.Generator().manual_seed(n + E)
    w = {"router": 3.0 * torch.randn(E, H, generator=g) / H ** 0.5, "router_bias": 0.5 * torch.randn(E, generator=g)}
    for e in range(E):
        w.update({f"gate_{e}": 2 * torch.randn(ff, H, generator=g) / H ** 0.5, f"up_{e}": 2 * torch.randn(ff, H, generator=g) / H ** 0.5,
                  f"down_{e}": torch.randn(H, ff, generator=g) / ff ** 0.5})
    if sff:
        w.update({"shared_gate": 2 * torch.randn(sff, H, generator=g) / H ** 0.5, "shared_up": 2 * torch.randn(sff, H, generator=g) / H ** 0.5,
                  "shared_down": torch.randn(H, sff, generator=g) / sff ** 0.5})
    w = {k: v.to(dtype) for k, v in w.items()}
    x = torch.randn(4 * n, H, generator=g).to(dtype)
    z = x.double() @ w["router"].double().T + w["router_bias"].double()
    zs = torch.sort(z, dim=1, descending=True).values
    clear = torch.ones(4 * n, dtype=torch.bool) if top == E else (zs[:, top - 1] - zs[:, top]) > 0.1
    x = x[clear][:n]
    n = x.shape[0]
    ff_part = _part(FEED_FORWARDS, "clamped_experts", {"hidden_size": H, "experts": E, "top": top, "ff": ff, "limit": 1.5,
                                                       "shared_ff": sff, "shared_limit": 0.8}, w, dtype)
    got = _sum_terms(ff_part.forward(x.to(DEV)))
    names = {"l.router": "router", "l.router.b": "router_bias", "l.shared.gate": "shared_gate", "l.shared.up": "shared_up",
             "l.shared.down": "shared_down"}
    names.update({f"l.e{e}.{m}": f"{m}_{e}" for e in range(E) for m in ("gate", "up", "down")})
    pw = {k: w[v].double() for k, v in names.items() if v in w}
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": 1.5}, "router": {"experts": E, "top": top}}
    if sff:
        mlp["shared"] = {"ff": sff, "limit": 0.8}
    want = plain.feed_forward(None, mlp, pw, "l.", x.double())
    _close(got, want, 1e-5 if dtype == torch.float32 else 2.5e-2, "clamped experts")
