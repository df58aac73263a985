"""The kernels behind the Dedelorn parts, each mechanism alone, against the plain implementation's function of
the same mechanism (float64 on the CPU), at sizes that are no powers of two, in float32 and (where the kernel has a
bfloat16 form) bfloat16.  Where random numbers would hide a fault (a key at a window's edge, a key far back in a
recurrent state, a page's border) the inputs are made so that it shows."""
import math

import pytest
import torch

from plain import dedelorn_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _ops():
    from zedinfer_amd import ops
    ops.load()
    return ops


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def _close(got, want, tol, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    err = float((got - want).abs().max())
    scale = max(1.0, float(want.abs().max()))
    assert err <= tol * scale, f"{what}: {err} of {scale}"


# ---- elementwise and the rotation ----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("act", ["silu", "gelu_tanh", "gelu_erf"])
def test_gated_activation(dtype, act):
    ops = _ops()
    g = torch.Generator().manual_seed(0)
    gu = (3 * torch.randn(7, 2 * 40 + 8, generator=g)).to(dtype)
    out = torch.empty(7, 40, dtype=dtype, device=DEV)
    d = gu.to(DEV)
    ops.gated_act(d[:, :40], d[:, 48:], act, out=out)                 # column slices of one product
    f = {"silu": plain.silu, "gelu_tanh": plain.gelu_tanh, "gelu_erf": plain.gelu_erf}[act]
    _close(out, f(gu[:, :40].double()) * gu[:, 48:].double(), 2e-6 if dtype == torch.float32 else 1e-2, act)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotation_of_neighbouring_pairs(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(1)
    n, heads, d, rot, base = 9, 3, 20, 12, 777.0
    x = torch.randn(n, heads * d, generator=g).to(dtype)
    pos = torch.tensor([0, 1, 2, 50, 51, 1000, 4095, 7, 8])
    inv = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device=DEV)
    table = ops.rope_table(_i32(pos.tolist()), inv)
    got = ops.rope_pairs(x.to(DEV).clone(), table, heads, d)
    want = plain.rotate_pairs(x.double().view(n, heads, d), pos, base, rot).view(n, heads * d)
    _close(got, want, 2e-4 if dtype == torch.float32 else 1e-2)       # float32 angles at position 4,095


# ---- latent attention ------------------------------------------------------------------------------------------------
def _paged(c, kr, page_size, pages, seed):
    """Put one sequence's latents into shuffled pages; returns the two caches and the block table."""
    T = c.shape[0]
    need = -(-T // page_size)
    perm = torch.randperm(pages, generator=torch.Generator().manual_seed(seed))[:need]
    cc = torch.full((pages, page_size, c.shape[1]), 9e3, dtype=c.dtype)          # what no table names is poison
    kk = torch.full((pages, page_size, kr.shape[1]), 9e3, dtype=kr.dtype)
    for j in range(T):
        cc[perm[j // page_size], j % page_size] = c[j]
        kk[perm[j // page_size], j % page_size] = kr[j]
    return cc.to(DEV), kk.to(DEV), perm.to(torch.int32)


def _plain_attend(qa, c, kr, pos, window, scale):
    """qa [n, H, rank + rot] at positions pos over the cached (c, kr) of one sequence."""
    rank = c.shape[1]
    out = torch.zeros(qa.shape[0], qa.shape[1], rank, dtype=torch.float64)
    for i, p in enumerate(pos):
        lo = max(0, p - window + 1) if window else 0
        keys = torch.cat([c[lo:p + 1], kr[lo:p + 1]], dim=1).double()
        for h in range(qa.shape[1]):
            s = torch.softmax((keys @ qa[i, h].double()) * scale, dim=0)
            out[i, h] = s @ c[lo:p + 1].double()
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window, page_size", [(0, 8), (13, 8), (16, 16), (17, 4), (64, 16), (150, 32)])
def test_latent_attention_sees_its_window_and_nothing_else(dtype, window, page_size):
    """Decoded tokens and a prompt's portion over shuffled pages.  For every query the key just inside the window
    is made to stand out, and the key just outside it twice as much: leaving the one out or letting the other
    in moves the result by its whole size.  Positions sit at page borders and beside them."""
    ops = _ops()
    g = torch.Generator().manual_seed(5)
    T, H, rank, rot, scale = 140, 3, 40, 6, 0.5
    c = (0.3 * torch.randn(T, rank, generator=g)).to(dtype)
    kr = (0.3 * torch.randn(T, rot, generator=g)).to(dtype)
    W = window if window else T + 1
    pos = [p for p in (0, 1, page_size - 1, page_size, page_size + 1, 63, 64, 65, W - 1, W, W + 1, 100, T - 1) if p < T]
    pos = sorted(set(pos))
    qa = torch.randn(len(pos), H, rank + rot, generator=g)
    for i, p in enumerate(pos):                    # planted keys, spaced so that each query has its own
        inside, outside = p - W + 1, p - W
        direction = qa[i, 0, :rank] / qa[i, 0, :rank].norm()
        if inside >= 0 and inside not in pos:
            c[inside] = (6.0 * direction).to(dtype)
        if outside >= 0 and window:
            c[outside] = (12.0 * direction).to(dtype)
    cc, kk, table = _paged(c, kr, page_size, 40, seed=window)
    want = _plain_attend(qa, c.float(), kr.float(), pos, window, scale)
    width = 12
    bt = torch.full((3, width if page_size * width >= T else -(-T // page_size)), -1, dtype=torch.int32)
    bt[1, :table.numel()] = table                  # the sequence is entry 1 of three
    out = torch.empty(len(pos), H, rank, dtype=torch.float32, device=DEV)
    ops.latent_attention(qa.to(DEV), cc, kk, _i32([1] * len(pos)), _i32(pos), bt.to(DEV), scale, window, out=out)
    _close(out, want, 2e-5 if dtype == torch.float32 else 2e-5, f"window {window}")     # the cache is given, sums are float32
    # some of the tokens only, through an index list
    some = [len(pos) - 1, 0, 3]
    out.fill_(float("nan"))
    ops.latent_attention(qa.to(DEV), cc, kk, _i32([1] * len(pos)), _i32(pos), bt.to(DEV), scale, window, out=out,
                         tok_index=_i32(some))
    _close(out[some], want[some], 2e-5, "listed tokens")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n, H, dim, rot, vdim, rank", [(11, 3, 20, 6, 28, 36), (11, 3, 24, 8, 28, 40), (70, 5, 128, 64, 48, 264)])
def test_latent_store_query_and_value_against_the_plain_mixer(dtype, n, H, dim, rot, vdim, rank):
    """The three kernels around the attention kernel: what is stored for a token is the normed latent and the
    turned key part, at the slot the step names (negative slots are skipped); the query carried through W_uk
    meets the latents as the plain query meets the keys made from them; values come out of W_uv."""
    ops = _ops()
    g = torch.Generator().manual_seed(7)
    base, eps, ps = 900.0, 1e-5, 4      # (sizes that are multiples of 8 go to the matrix cores in bfloat16)
    pos = torch.arange(20, 20 + n)
    dkv = torch.randn(n, rank + rot, generator=g)
    gain = 1 + 0.2 * torch.randn(rank, generator=g)
    q = torch.randn(n, H * (dim + rot), generator=g).to(dtype)
    w_uk = (torch.randn(H * dim, rank, generator=g) / rank ** 0.5).to(dtype)
    w_uv = (torch.randn(H * vdim, rank, generator=g) / rank ** 0.5).to(dtype)
    inv = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device=DEV)
    table = ops.rope_table(_i32(pos.tolist()), inv)
    slots = list(range(37, 37 + n))
    slots[4] = -1
    cc = torch.zeros(40, ps, rank, dtype=dtype, device=DEV)
    kk = torch.zeros(40, ps, rot, dtype=dtype, device=DEV)
    ops.latent_store(dkv.to(DEV), gain.to(dtype).to(DEV), eps, table, _i32(slots), cc, kk, rank, rot)
    c_want = plain.rms(dkv[:, :rank].double(), eps) * gain.to(dtype).double()
    kr_want = plain.rotate_pairs(dkv[:, rank:].double(), pos, base, rot)
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    for i, s in enumerate(slots):
        if s >= 0:
            _close(cc.view(-1, rank)[s], c_want[i], tol, "latent")
            _close(kk.view(-1, rot)[s], kr_want[i], tol, "key part")
    assert float(cc.view(-1, rank)[37 + 4].abs().max()) == 0.0 and float(cc.view(-1, rank)[:37].abs().max()) == 0.0
    qa = torch.empty(n, H, rank + rot, dtype=torch.float32, device=DEV)
    q32 = q.float()        # the mixer's projection leaves float32
    uk_t = w_uk.view(H, dim, rank).transpose(1, 2).contiguous().to(DEV) if dtype == torch.bfloat16 and dim % 8 == 0 else None
    ops.latent_query(q32.to(DEV), w_uk.to(DEV), table, H, dim, rank, rot, out=qa, w_uk_t=uk_t)
    qd = q.double().view(n, H, dim + rot)
    c_any = torch.randn(rank, generator=g).double()
    for h in range(H):
        k_plain = w_uk.double()[h * dim:(h + 1) * dim] @ c_any                         # the key the plain mixer makes
        _close(qa[:, h, :rank].double().cpu() @ c_any, qd[:, h, :dim] @ k_plain, 3e-5 if uk_t is None else 1e-2, "carried query")
    _close(qa[:, :, rank:], plain.rotate_pairs(qd[..., dim:], pos, base, rot), 3e-5 if dtype == torch.float32 else 3e-5, "turned query")
    o = torch.randn(n, H, rank, generator=g)
    out = torch.empty(n, H * vdim, dtype=dtype, device=DEV)
    ops.latent_value(o.to(DEV), w_uv.to(DEV), vdim, out=out)
    want = torch.stack([o[:, h].double() @ w_uv.double()[h * vdim:(h + 1) * vdim].t() for h in range(H)], 1).reshape(n, H * vdim)
    _close(out, want, 2e-5 if dtype == torch.float32 else 1e-2, "values")


# ---- the gated delta rule ---------------------------------------------------------------------------------------------
DELTA_SIZES = [(6, 2, 24, 40, 4), (3, 3, 72, 20, 3), (4, 1, 8, 72, 5), (2, 2, 130, 16, 1), (1, 1, 33, 17, 2)]


def _delta_inputs(n, heads, kvh, dim, vdim, taps, seed):
    g = torch.Generator().manual_seed(seed)
    C = 2 * kvh * dim + heads * vdim
    proj = torch.randn(n, C + heads * vdim + 2 * heads, generator=g)
    conv = 0.6 * torch.randn(C, taps, generator=g)
    a_log, dt_bias = 0.5 * torch.randn(heads, generator=g), 0.5 * torch.randn(heads, generator=g)
    return proj, conv, a_log, dt_bias


def _plain_prepare(proj, conv, a_log, dt_bias, heads, kvh, dim, vdim):
    """The plain mixer's steps up to the recurrence, for one whole sequence."""
    n, C = proj.shape[0], 2 * kvh * dim + heads * vdim
    x = plain.silu(plain.short_conv(proj[:, :C].double(), conv.double()))
    q = x[:, :kvh * dim].view(n, kvh, dim)
    k = x[:, kvh * dim:2 * kvh * dim].view(n, kvh, dim)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    b, a = proj[:, C + heads * vdim:C + heads * vdim + heads].double(), proj[:, C + heads * vdim + heads:].double()
    beta = torch.sigmoid(b)
    decay = torch.exp(-torch.exp(a_log.double()) * plain.softplus(a + dt_bias.double()))
    return q, k, x[:, 2 * kvh * dim:].view(n, heads, vdim), beta, decay


@pytest.mark.parametrize("heads, kvh, dim, vdim, taps", DELTA_SIZES)
@pytest.mark.parametrize("cuts", [[57], [1] * 9 + [48], [2, 3, 1, 1, 20, 2, 28], [50, 7]])
def test_delta_rule_in_portions_equals_the_plain_recurrence(heads, kvh, dim, vdim, taps, cuts):
    """One sequence fed in portions (down to one token, shorter than the convolution) through a state slot that held
    another sequence before: convolution tail and matrix state carry over, and a fresh request starts from zero."""
    ops = _ops()
    n = sum(cuts)
    proj, conv, a_log, dt_bias = _delta_inputs(n, heads, kvh, dim, vdim, taps, seed=dim + taps)
    q, k, v, beta, decay = _plain_prepare(proj, conv, a_log, dt_bias, heads, kvh, dim, vdim)
    want = torch.stack([plain.delta_rule(q[:, h // (heads // kvh)], k[:, h // (heads // kvh)], v[:, h], beta[:, h], decay[:, h])
                        for h in range(heads)], 1)
    floats = ops.delta_state_floats(heads, dim, vdim, kvh, taps)
    state = torch.randn(3, floats, device=DEV)                      # slots 0 and 2 belong to others
    before = state.clone()
    state[1].zero_()                                               # what admission does
    dev = [t.to(DEV) for t in (proj, conv, a_log, dt_bias)]
    got, at = [], 0
    for c in cuts:
        rows = dev[0][at:at + c].contiguous()
        qk = torch.empty(c, 2 * kvh * dim, device=DEV)
        vv = torch.empty(c, heads * vdim, device=DEV)
        bg = torch.empty(c, 2, heads, device=DEV)
        es, el, slot, seq = _i32([0]), _i32([c]), _i32([1]), _i32([0] * c)
        ops.delta_prepare(rows, dev[1], dev[2], dev[3], state, seq, es, slot, heads, kvh, dim, vdim, taps, qk, vv, bg)
        ops.delta_conv_state(state, rows, es, el, slot, heads, kvh, dim, vdim, taps)
        out = torch.empty(c, heads * vdim, device=DEV)
        ops.delta_rule(qk, vv, bg, state, es, el, slot, heads, kvh, dim, vdim, out=out)
        got.append(out.cpu())
        if at == 0:
            _close(qk[:, :kvh * dim].view(c, kvh, dim), q[:c], 2e-5, "q")
            _close(qk[:, kvh * dim:].view(c, kvh, dim), k[:c], 2e-5, "k")
            _close(bg[:, 0], beta[:c], 2e-5, "beta")
            _close(bg[:, 1], decay[:c], 2e-5, "decay")
        at += c
    _close(torch.cat(got).view(n, heads, vdim), want, 5e-5, "read-out")
    assert torch.equal(state[0], before[0]) and torch.equal(state[2], before[2])
    C = 2 * kvh * dim + heads * vdim
    if taps > 1:                                                    # the tail is the sequence's last taps - 1 rows
        tail = state[1, heads * dim * vdim:heads * dim * vdim + (taps - 1) * C].view(taps - 1, C).cpu()
        assert torch.equal(tail, proj[n - (taps - 1):, :C])


def test_delta_rule_keeps_a_key_written_far_back_and_entries_do_not_mix():
    """Three entries in one launch, unequal, in slots out of order.  In entry 1 the first token writes a value under a
    key that no later token touches (decays of 1); 300 tokens on, a query with that key must read the value back."""
    ops = _ops()
    g = torch.Generator().manual_seed(11)
    heads, kvh, dim, vdim = 2, 1, 16, 24
    lens = [5, 301, 1]
    n = sum(lens)
    qk = torch.zeros(n, 2 * dim)
    k = torch.randn(n, dim, generator=g)
    k[:, 0] = 0.0                                                   # nobody else touches direction 0
    k = k / k.norm(dim=1, keepdim=True)
    q = torch.randn(n, dim, generator=g)
    v = torch.randn(n, heads * vdim, generator=g)
    bg = torch.rand(n, 2, heads, generator=g)
    first, last = lens[0], lens[0] + lens[1] - 1
    bg[first:last + 1, 1] = 1.0                                     # entry 1 forgets nothing
    k[first] = 0.0
    k[first, 0] = 1.0
    bg[first, 0] = 1.0
    q[last] = 0.0
    q[last, 0] = 1.0
    qk[:, :dim], qk[:, dim:] = q, k
    state = torch.zeros(4, heads * dim * vdim, device=DEV)
    out = torch.empty(n, heads * vdim, device=DEV)
    ops.delta_rule(qk.to(DEV), v.to(DEV), bg.to(DEV), state, _i32([0, 5, 306]), _i32(lens), _i32([3, 0, 2]), heads, kvh, dim,
                   vdim, out=out)
    _close(out[last], v[first], 1e-5, "the far key")
    at = 0
    for ln in lens:                                                 # every entry alone gives the same
        want = torch.stack([plain.delta_rule(q[at:at + ln].double(), k[at:at + ln].double(),
                                             v[at:at + ln, h * vdim:(h + 1) * vdim].double(), bg[at:at + ln, 0, h].double(),
                                             bg[at:at + ln, 1, h].double()) for h in range(heads)], 1).reshape(ln, -1)
        _close(out[at:at + ln], want, 5e-5, "entry")
        at += ln
    assert float(state[1].abs().max()) == 0.0                       # the slot nobody holds


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_rms_norm(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(13)
    n, heads, vdim, eps = 6, 3, 28, 1e-3
    o = 5 * torch.randn(n, heads * vdim, generator=g)
    w = 1 + 0.3 * torch.randn(vdim, generator=g)
    gate = torch.randn(n, heads * vdim + 10, generator=g)
    out = torch.empty(n, heads * vdim, dtype=dtype, device=DEV)
    ops.gated_rms_norm(o.to(DEV), w.to(DEV), gate.to(DEV)[:, 10:], heads, vdim, eps, out=out)
    want = (plain.rms(o.double().view(n, heads, vdim), eps) * w.double() * plain.silu(gate[:, 10:].double().view(n, heads, vdim)))
    _close(out, want.view(n, -1), 2e-5 if dtype == torch.float32 else 1e-2)


# ---- routed experts ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("experts, top", [(12, 4), (5, 1), (3, 3), (70, 6), (200, 2)])
def test_router_choice_and_weights(experts, top):
    ops = _ops()
    g = torch.Generator().manual_seed(experts)
    n, scale = 37, 1.7
    z = 2 * torch.randn(n, experts, generator=g)
    z[3, :] = 0.25                                                   # all equal: the lowest indices win
    corr = 0.05 * torch.randn(experts, generator=g)
    corr_flat = corr.clone()
    idx = torch.empty(n, top, dtype=torch.int32, device=DEV)
    wt = torch.empty(n, top, dtype=torch.float32, device=DEV)
    ops.moe_route(z.to(DEV), corr.to(DEV), top, scale, idx, wt)
    s = torch.softmax(z.double(), -1)
    choice = s + corr_flat.double()
    for t in range(n):
        order = sorted(range(experts), key=lambda e: (-float(choice[t, e]), e))[:top]
        got = idx[t].tolist()
        if t == 3:
            want3 = sorted(range(experts), key=lambda e: (-float(corr_flat[e]), e))[:top]
            assert got == want3
        # a near-tie may be ordered either way in float32; the chosen set and each chosen expert's weight must hold
        margin = float(choice[t, order[-1]] - sorted(choice[t].tolist(), reverse=True)[top]) if top < experts else 1.0
        if margin > 1e-6:
            assert sorted(got) == sorted(order), (t, got, order)
        for j, e in enumerate(got):
            assert abs(float(wt[t, j]) - scale * float(s[t, e])) <= 2e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n, experts, top, H, ff", [(1, 6, 3, 80, 56), (23, 6, 3, 80, 56), (300, 5, 1, 64, 40),
                                                    (130, 3, 3, 84, 36), (700, 4, 2, 64, 72)])
def test_experts_products_over_the_sorted_pairs(dtype, n, experts, top, H, ff):
    """Grouping, the two products (every tile size the part would choose) and the weighted sum against a loop over
    tokens and their experts; an expert that nobody chooses is among them."""
    ops = _ops()
    g = torch.Generator().manual_seed(n + experts)
    x = torch.randn(n, H, generator=g).to(dtype)
    up = (torch.randn(experts, ff, H, generator=g) / H ** 0.5).to(dtype)
    down = (torch.randn(experts, H, ff, generator=g) / ff ** 0.5).to(dtype)
    idx = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(n)]).to(torch.int32)
    if experts > top:
        idx[idx == experts - 1] = 0 if top == 1 else idx[idx == experts - 1]       # with one choice: the last expert idles
    wt = torch.rand(n, top, generator=g)
    pairs = n * top
    rows = ops.moe_tile_rows(dtype, dtype, (H, ff), pairs, experts)
    tiles = ops.moe_max_tiles(pairs, experts, rows)
    plan = torch.zeros(1 + 3 * tiles, dtype=torch.int32, device=DEV)
    order = torch.empty(pairs, dtype=torch.int32, device=DEV)
    place = torch.empty(pairs, dtype=torch.int32, device=DEV)
    ops.moe_group(idx.to(DEV), experts, rows, plan, order, place)
    flat = idx.view(-1)
    o = order.cpu().long()
    assert sorted(o.tolist()) == list(range(pairs)) and torch.equal(place.cpu().long()[o], torch.arange(pairs))
    assert (flat[o][1:] >= flat[o][:-1]).all()                                     # expert by expert
    used = int(plan[0])
    assert used == sum(-(-int((flat == e).sum()) // rows) for e in range(experts)) <= tiles
    act = torch.empty(pairs, ff, dtype=dtype, device=DEV)
    ops.moe_linear(x.to(DEV), up.to(DEV), plan, rows, tiles, out=act, source=order, source_div=top, activation="gelu_erf")
    y = torch.empty(pairs, H, dtype=torch.float32, device=DEV)
    ops.moe_linear(act, down.to(DEV), plan, rows, tiles, out=y)
    out = torch.empty(n, H, dtype=torch.float32, device=DEV)
    ops.moe_combine(y, wt.to(DEV), place, out)
    want = torch.zeros(n, H, dtype=torch.float64)
    for t in range(n):
        for j in range(top):
            e = int(idx[t, j])
            want[t] += float(wt[t, j]) * (plain.gelu_erf(x[t].double() @ up[e].double().t()) @ down[e].double().t())
    _close(out, want, 3e-5 if dtype == torch.float32 else 2e-2, "experts")


@pytest.mark.parametrize("rank, rot", [(40, 8), (136, 24), (264, 16)])
@pytest.mark.parametrize("window, page_size", [(0, 8), (13, 8), (64, 16), (150, 4)])
@pytest.mark.parametrize("waves, chunk_keys", [(1, 0), (4, 0), (1, 128), (4, 128)])
def test_latent_attention_on_the_matrix_cores(rank, rot, window, page_size, waves, chunk_keys):
    """A prompt's portion of 37 tokens (tiles that end inside a token's heads, and a last tile with rows to spare)
    beside a decoded token of another sequence, over shuffled pages of one pool; every cut of the keys and both
    workgroup sizes against the plain sums; the keys at the window's edge planted as for the plain kernel."""
    ops = _ops()
    if chunk_keys and not window:
        pytest.skip("keys are cut only under a window")
    g = torch.Generator().manual_seed(rank + window)
    H, scale, dtype = 5, 0.5, torch.bfloat16
    T = [140, 77]
    c = [(0.3 * torch.randn(t, rank, generator=g)).to(dtype) for t in T]
    kr = [(0.3 * torch.randn(t, rot, generator=g)).to(dtype) for t in T]
    past, lens = [103, 76], [37, 1]
    n = sum(lens)
    qa = torch.randn(n, H, rank + rot, generator=g)
    W = window if window else 10 ** 6
    for e, row in ((0, 36), (1, 37)):                               # the last token of either entry
        p = past[e] + lens[e] - 1
        direction = qa[row, 0, :rank] / qa[row, 0, :rank].norm()
        if p - W + 1 >= 0:
            c[e][p - W + 1] = (6.0 * direction).to(dtype)
        if p - W >= 0:
            c[e][p - W] = (12.0 * direction).to(dtype)
    pages = 80
    perm = torch.randperm(pages, generator=g)
    cc = torch.full((pages, page_size, rank), 9e3, dtype=dtype)
    kk = torch.full((pages, page_size, rot), 9e3, dtype=dtype)
    width = -(-max(T) // page_size) + 3
    bt = torch.full((2, width), -1, dtype=torch.int32)
    at = 0
    for e in range(2):
        for j in range(T[e]):
            if j % page_size == 0:
                bt[e, j // page_size] = perm[at]
                at += 1
            cc[bt[e, j // page_size], j % page_size] = c[e][j]
            kk[bt[e, j // page_size], j % page_size] = kr[e][j]
    want = torch.cat([_plain_attend(qa[:37].to(dtype).float(), c[0].float(), kr[0].float(), list(range(103, 140)), window, scale),
                      _plain_attend(qa[37:].to(dtype).float(), c[1].float(), kr[1].float(), [76], window, scale)])
    chunks = 1
    if chunk_keys:
        chunks = -(-(window + -(-16 * waves // H) + 1) // chunk_keys)
        if chunks == 1:
            chunk_keys = 0
    need = ops.latent_attention_cores_workspace(n, H, rank, chunks)
    ws = torch.full((max(need, 1),), float("nan"), device=DEV)
    out = torch.full((n, H, rank), float("nan"), device=DEV)
    ops.latent_attention_cores(qa.to(DEV), cc.to(DEV), kk.to(DEV), _i32([0, 37]), _i32(lens), _i32(past), bt.to(DEV), scale,
                               window, out=out, waves=waves, chunk_keys=chunk_keys, chunks=chunks, workspace=ws)
    _close(out, want, 1.5e-2, f"rank {rank} window {window} waves {waves} chunks {chunks}")
    # and against the plain kernel on the same cache
    plain_out = torch.empty_like(out)
    ops.latent_attention(qa.to(DEV), cc.to(DEV), kk.to(DEV), _i32([0] * 37 + [1]), _i32(list(range(103, 140)) + [76]),
                         bt.to(DEV), scale, window, out=plain_out)
    _close(out, plain_out, 1.5e-2, "against the plain kernel")


def test_latent_attention_cores_plan_is_a_function_of_the_shape():
    ops = _ops()
    assert ops.latent_attention_cores_plan(2048, 1, 12, 1024, 256) == (4, 0, 1)          # a prompt fills the chip uncut
    waves, keys, chunks = ops.latent_attention_cores_plan(8, 8, 12, 1024, 256)           # decoded tokens: cut
    assert waves == 1 and keys == ops.mixing.LATENT_CHUNK_KEYS and chunks * keys >= 1024 + 3
    assert ops.latent_attention_cores_plan(8, 8, 12, 0, 256) == (1, 0, 1)                # no window, no cut
    assert ops.latent_attention_cores_plan(8, 8, 12, 72, 256) == (1, 0, 1)               # a window of one chunk
