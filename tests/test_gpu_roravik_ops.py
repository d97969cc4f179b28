"""Each mechanism of the Roravik layers alone, kernel against the plain functions: the two recurrences carried
through pieces and slots (decays that forget nothing and everything), the rotation inside a 32-bit matrix, the mixes
with the previous token's input, the convolution on q, k and v carried through pieces, the window's edge with one key
made to stand out just inside and just outside it under a soft cap and a learned sink (prompt and single-token
kernels, at page borders, plain and matrix-core kernels), the head norm with a silu gate, the choice of experts with a
correction and groups scored by their two best, the gated row sum, the weighted sum and the soft cap."""

import pytest
import torch

from tests.plain import roravik_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PAGE = 64
D64 = torch.float64


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _close(got, want, tol, what=""):
    want = want.to(D64)
    err = float((got.detach().cpu().to(D64) - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err < tol, f"{what}: {err:.3g} >= {tol}"


def _i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def _pieces(lengths, cuts):
    """Steps that bring sequence ``b`` in pieces: for every step the (sequence, first, count) triples."""
    at = [0] * len(lengths)
    steps = []
    while any(a < n for a, n in zip(at, lengths)):
        step = []
        for b, n in enumerate(lengths):
            if at[b] < n:
                c = min(cuts[(len(steps) + b) % len(cuts)], n - at[b])
                step.append((b, at[b], c))
                at[b] += c
        steps.append(step)
    return steps


@pytest.mark.parametrize("dk,dv", [(1, 12), (6, 1), (17, 9), (20, 36), (64, 64), (128, 32), (256, 16)])
@pytest.mark.parametrize("bonus,logits", [(False, False), (True, False), (True, True)])
def test_recurrences_through_pieces_and_slots(dk, dv, bonus, logits):
    """Three sequences of unequal length in slots of their own beside slots of others, brought in pieces of 1 to 40
    tokens; a head that forgets nothing and one that keeps nothing."""
    from rocml_amd import ops
    g = _gen(dk * 100 + dv + bonus)
    H, lengths = 3, [70, 5, 33]
    T = sum(lengths)
    q, k = torch.randn(T, H, dk, generator=g, dtype=D64), torch.randn(T, H, dk, generator=g, dtype=D64) / dk ** 0.5
    v = torch.randn(T, H, dv, generator=g, dtype=D64)
    starts = [0, 70, 75]
    if bonus:
        w = torch.rand(T, H, dk, generator=g, dtype=D64)
        w[:, 0] = 1.0
        w[:, 1] = 0.0
        u = torch.randn(H, dk, generator=g, dtype=D64)
        offset = torch.randn(H, dk, generator=g, dtype=D64)
        want = torch.cat([plain.recurrence_read_before(q[s:s + n], k[s:s + n], v[s:s + n], w[s:s + n], u) for s, n in zip(starts, lengths)])
    else:
        decay = [1.0, 0.0, 0.93]
        want = torch.cat([plain.recurrence_read_after(q[s:s + n], k[s:s + n], v[s:s + n], decay) for s, n in zip(starts, lengths)])
    slots = [4, 0, 2]
    state = torch.zeros(6, H, dv, dk, dtype=torch.float32, device=DEV)
    state[1].fill_(7.0)        # a slot of somebody else
    got = torch.zeros(T, H * dv, dtype=torch.float32)
    for step in _pieces(lengths, [1, 40, 2, 7]):
        rows = [i for b, first, c in step for i in range(starts[b] + first, starts[b] + first + c)]
        cu = [0]
        for _, _, c in step:
            cu.append(cu[-1] + c)
        # q, k, v side by side in one matrix with a few columns in front, as a projection has them
        mat = torch.cat([torch.zeros(len(rows), 3, dtype=D64), q[rows].reshape(len(rows), -1), k[rows].reshape(len(rows), -1),
                         v[rows].reshape(len(rows), -1)], dim=1).float().to(DEV).contiguous()
        out = torch.empty(len(rows), H * dv, dtype=torch.float32, device=DEV)
        kw = dict(decay=w[rows].reshape(len(rows), -1).float().to(DEV).contiguous(), bonus=u.reshape(-1).float().to(DEV)) if bonus \
            else dict(head_decay=torch.tensor(decay, dtype=torch.float32, device=DEV))
        if bonus and logits:
            # the decays as logits x with an offset: w = exp(-exp(x + offset)); the heads that forget nothing and everything
            # get logits far below and far above zero
            x = torch.log(-torch.log(w[rows].clamp(1e-30, 1 - 1e-12))).clamp(-40.0, 40.0) - offset
            kw.update(decay=x.reshape(len(rows), -1).float().to(DEV).contiguous(), decay_offset=offset.reshape(-1).float().to(DEV))
        ops.decay_scan(mat, 3, mat, 3 + H * dk, mat, 3 + 2 * H * dk, state, _i32(cu), _i32([slots[b] for b, _, _ in step]), out,
                       H, dk, dv, **kw)
        got[rows] = out.cpu()
    _close(got, want.reshape(T, -1), 2e-4 if logits else 2e-5, "recurrence")
    assert float((state[1] - 7.0).abs().max()) == 0.0 and float(state[3].abs().max()) == 0.0, "other slots stay as they were"


@pytest.mark.parametrize("d,rot", [(8, 8), (20, 4), (12, 0), (64, 32), (6, 2)])
def test_rotation_inside_a_matrix(d, rot):
    from rocml_amd import ops
    g = _gen(d + rot)
    T, H = 9, 3
    x = torch.randn(T, H, d, generator=g, dtype=D64)
    pos = torch.tensor([0, 1, 2, 63, 64, 65, 1000, 4097, 30000])
    base = 777.0
    want = (plain.rotate(x, pos, {"dims": rot, "base": base}) if rot else x) * 0.37
    want[:, 2] *= 1.9 / 0.37          # the last head has a scale of its own
    mat = torch.cat([torch.ones(T, 5, dtype=D64), x.reshape(T, -1), torch.ones(T, 2, dtype=D64)], dim=1).float().to(DEV).contiguous()
    cos = sin = None
    if rot:
        f = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=D64, device=DEV)
        cos = torch.empty(T, rot // 2, dtype=torch.float32, device=DEV)
        sin = torch.empty_like(cos)
        ops.rope_table(pos.to(torch.int32).to(DEV), f, cos, sin)
    ops.rotate_rows(mat, 5, H, d, rot, cos, sin, 0.37, heads_first=2, scale_rest=1.9)
    _close(mat[:, 5:5 + H * d], want.reshape(T, -1), 2e-6, "rotated heads")
    assert float((mat[:, :5] - 1).abs().max()) == 0.0 and float((mat[:, 5 + H * d:] - 1).abs().max()) == 0.0


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("n", [5, 72, 130])
def test_mixes_with_the_previous_token(n, dtype, tol):
    from rocml_amd import ops
    g = _gen(n)
    lengths, starts, slots = [40, 3, 1], [0, 40, 43], [2, 5, 0]
    T = sum(lengths)
    h = torch.randn(T, n, generator=g).to(dtype)
    mu = torch.rand(5, n, generator=g)
    want = []
    for s, c in zip(starts, lengths):
        x = h[s:s + c].double()
        prev = torch.cat([torch.zeros(1, n, dtype=D64), x[:-1]])
        want.append(torch.stack([x + (prev - x) * mu[m].double() for m in range(5)]))
    want = torch.cat(want, dim=1)
    state = torch.zeros(6, n, dtype=torch.float32, device=DEV)
    state[1].fill_(3.0)
    got = torch.zeros(5, T, n, dtype=torch.float32)
    for step in _pieces(lengths, [1, 17, 2]):
        rows = [i for b, first, c in step for i in range(starts[b] + first, starts[b] + first + c)]
        cu, seq = [0], []
        for j, (_, _, c) in enumerate(step):
            cu.append(cu[-1] + c)
            seq += [j] * c
        out = torch.empty(5, len(rows), n, dtype=dtype, device=DEV)
        ops.shift_mix(h[rows].to(DEV).contiguous(), mu.to(DEV), state, _i32(seq), _i32(cu), _i32([slots[b] for b, _, _ in step]), out)
        got[:, rows] = out.float().cpu()
    _close(got, want, tol, "mixes")
    assert float((state[1] - 3.0).abs().max()) == 0.0
    assert torch.equal(state[2].cpu(), h[39].float()) and torch.equal(state[0].cpu(), h[43].float()), "the kept row is the last one"


@pytest.mark.parametrize("taps", [1, 2, 4, 8])
def test_convolution_without_bias_through_pieces(taps):
    from rocml_amd import ops
    g = _gen(taps)
    C, lengths, starts, slots = 22, [50, 2, 9], [0, 50, 52], [1, 3, 0]
    T = sum(lengths)
    u = torch.randn(T, C, generator=g, dtype=D64)
    w = torch.randn(C, taps, generator=g, dtype=D64)
    want = torch.cat([plain.short_conv(u[s:s + n], w) for s, n in zip(starts, lengths)])
    state = torch.zeros(4, max(taps - 1, 0), C, dtype=torch.float32, device=DEV)
    got = torch.zeros(T, C, dtype=torch.float32)
    for step in _pieces(lengths, [1, 2, 30, 1, 5]):
        rows = [i for b, first, c in step for i in range(starts[b] + first, starts[b] + first + c)]
        cu, seq = [0], []
        for j, (_, _, c) in enumerate(step):
            cu.append(cu[-1] + c)
            seq += [j] * c
        mat = torch.cat([torch.zeros(len(rows), 4, dtype=D64), u[rows]], dim=1).float().to(DEV).contiguous()
        out = torch.empty(len(rows), C, dtype=torch.float32, device=DEV)
        ops.causal_conv(mat, 4, C, w.t().float().contiguous().to(DEV), None, state, _i32(seq), _i32(cu), _i32([slots[b] for b, _, _ in step]),
                        out, silu=False)
        got[rows] = out.cpu()
    _close(got, want, 2e-6, "convolution")


def _attend(q, k, v, dtype, scale, cap, window, sink, decode_from, perm_seed):
    """``q [T, H, d]``, ``k [T, G, d]``, ``v [T, G, dv]`` of one sequence through the append kernel and the attention: the first
    ``decode_from`` positions as one prompt step, the rest one token a step.  The sequence's pages lie scattered in the pool."""
    from rocml_amd import ops
    T, H, d = q.shape
    G, dv = k.shape[1], v.shape[-1]
    n_pages = (T + PAGE - 1) // PAGE
    perm = torch.randperm(n_pages + 3, generator=_gen(perm_seed))[:n_pages]
    kc = torch.zeros(n_pages + 3, G, PAGE, d, dtype=dtype, device=DEV)
    vc = torch.zeros(n_pages + 3, G, dv, PAGE, dtype=dtype, device=DEV)
    table = perm.to(torch.int32).reshape(1, -1).to(DEV)
    out = torch.zeros(T, H * dv, dtype=torch.float32)
    steps = [(0, decode_from)] + [(i, 1) for i in range(decode_from, T)]
    for first, n in steps:
        if n == 0:
            continue
        rows = slice(first, first + n)
        qkv = torch.cat([q[rows].reshape(n, -1), k[rows].reshape(n, -1), v[rows].reshape(n, -1)], dim=1).float().to(DEV).contiguous()
        seq, pos = _i32([0] * n), _i32(list(range(first, first + n)))
        qo = torch.empty(n, H * d, dtype=dtype, device=DEV)
        ops.qk_norm_rope_append(qkv, H, G, d, None, None, 1.0, None, None, 0, qo, kc, vc, table, seq, pos, v_head_dim=dv)
        o = torch.empty(n, H * dv, dtype=dtype, device=DEV)
        ws = torch.empty(1 << 22, dtype=torch.uint8, device=DEV)
        ops.attention(qo, o, kc, vc, table, seq, pos, H, G, d, scale, window, workspace=ws, cu_seqlens=_i32([0, n]), max_new=n,
                      q_counts=[n], max_len=first + n, n_splits=ops.decode_splits(G, 256, n_pages) if n == 1 else 0,
                      v_head_dim=dv, sink=True, sinks=sink.float().to(DEV), softcap=cap)
        out[rows] = o.float().cpu()
    return out


@pytest.mark.parametrize("dtype,H,G,d,dv", [(torch.float32, 4, 2, 24, 16), (torch.float32, 2, 2, 64, 64), (torch.bfloat16, 4, 2, 64, 64),
                                            (torch.bfloat16, 8, 1, 128, 128), (torch.bfloat16, 3, 3, 16, 40), (torch.bfloat16, 6, 2, 96, 96),
                                            (torch.bfloat16, 2, 1, 256, 256), (torch.bfloat16, 4, 4, 32, 32), (torch.bfloat16, 4, 2, 192, 192),
                                            (torch.bfloat16, 34, 2, 64, 64)])
@pytest.mark.parametrize("window", [1, 5, 64, 65, 130])
def test_window_edge_under_a_soft_cap_and_a_sink(dtype, H, G, d, dv, window):
    """One key is made to win by far: just inside the window it takes the whole output, just outside it nothing of it shows,
    for queries in the prompt and for decoded ones, with the window's edge before, on and after page borders.  The cap bounds
    the winner's score, so the sink (equal to the cap in one head, far below in the others) takes half of that head's weight."""
    g = _gen(window * 7 + d)
    T, decode_from = 200, 150
    scale, cap = 1.7 / d ** 0.5, 6.0
    q = torch.randn(T, H, d, generator=g, dtype=D64)
    k = torch.randn(T, G, d, generator=g, dtype=D64)
    v = torch.randn(T, G, dv, generator=g, dtype=D64)
    sink = torch.full((H,), -20.0, dtype=D64)
    sink[0] = cap
    for i in (70, 127, 128, 140, 160, 191, 192, 199):       # queries in the prompt and decoded ones
        for j in (i - window + 1, i - window):                # just inside, just outside
            if j >= 0:
                k[j] = 0.0
        inside = i - window + 1
        if inside >= 0:
            k[inside, :] = 30.0 * q[i, ::H // G] / q[i, ::H // G].norm(dim=-1, keepdim=True)
        if inside - 1 >= 0 and window > 1:
            k[inside - 1, :] = 40.0 * q[i, ::H // G] / q[i, ::H // G].norm(dim=-1, keepdim=True)
    if dtype == torch.bfloat16:
        q, k, v = (t.to(torch.bfloat16).double() for t in (q, k, v))
    want = plain.capped_window_softmax(q, k, v, scale, cap, window, sink).reshape(T, -1)
    got = _attend(q, k, v, dtype, scale, cap, window, sink, decode_from, window)
    _close(got, want, 2e-5 if dtype == torch.float32 else 3e-2, f"window {window}")
    # and the edge shows: without the key just inside, the output of such a query is another one
    i = 160
    if i - window + 1 >= 0 and window > 1:
        k2 = k.clone()
        k2[i - window + 1] = 0.0
        other = plain.capped_window_softmax(q, k2, v, scale, cap, window, sink).reshape(T, -1)
        assert float((other[i] - want[i]).abs().max()) > 0.1


@pytest.mark.parametrize("heads,dv", [(1, 1), (3, 17), (4, 64), (2, 130)])
def test_head_norm_with_a_silu_gate(heads, dv):
    from rocml_amd import ops
    g = _gen(heads + dv)
    T, eps = 6, 1e-3
    o = torch.randn(T, heads, dv, generator=g, dtype=D64) * 4
    gate = torch.randn(T, heads * dv, generator=g, dtype=D64) * 2
    gain = 1 + 0.3 * torch.randn(heads * dv, generator=g, dtype=D64)
    mat = torch.cat([torch.zeros(T, 3, dtype=D64), gate], dim=1).float().to(DEV).contiguous()
    for with_gain in (True, False):
        want = plain.rms(o, eps).reshape(T, -1) * (gain if with_gain else 1.0) * plain.silu(gate)
        for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
            out = torch.empty(T, heads * dv, dtype=dtype, device=DEV)
            ops.head_norm_gate(o.reshape(T, -1).float().to(DEV), mat, 3, gain.float().to(DEV) if with_gain else None, out, heads, eps,
                               gate="silu")
            _close(out, want, tol, f"gain {with_gain}")


@pytest.mark.parametrize("experts,top,groups", [(8, 3, (2, 1)), (6, 2, (3, 2)), (6, 3, None), (4, 2, (4, 2)), (2, 2, (1, 1)), (1, 1, None),
                                                (64, 6, (8, 3)), (130, 5, (10, 4))])
def test_choice_of_experts_with_a_correction(experts, top, groups):
    """Scores by sigmoid, a correction that changes the choice and not the weights (large enough to make choice scores
    negative and to move whole groups), groups scored by the sum of their two best."""
    from rocml_amd import ops
    g = _gen(experts * 10 + top)
    T = 300
    z = torch.randn(T, experts, generator=g) * 2.0
    corr = torch.randn(experts, generator=g) * 0.7 - 1.0
    router = {"top": top, "groups": None if groups is None else {"count": groups[0], "keep": groups[1]}}
    want_e, want_w = plain.choose_experts(z.double(), corr.double(), router)
    # the logits as the leading columns of a wider matrix
    wide = torch.cat([z, torch.full((T, 1), 9.0)], dim=1).to(DEV).contiguous()
    chosen = torch.empty(T, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(T, top, dtype=torch.float32, device=DEV)
    ops.moe_route(wide[:, :experts], top, groups, 1e-20, chosen, weight, sigmoid=True, correction=corr.to(DEV), group_top2=True)
    assert torch.equal(chosen.cpu().long(), want_e)
    _close(weight, want_w, 1e-5, "weights")
    if groups is not None and groups[1] < groups[0] and experts // groups[0] > 1:
        by_max = torch.empty_like(chosen)
        ops.moe_route(wide[:, :experts], top, groups, 1e-20, by_max, weight, sigmoid=True, correction=corr.to(DEV), group_top2=False)
        assert not torch.equal(by_max.cpu(), chosen.cpu()), "the two ways to score a group differ on some token"


def test_softmax_routing_is_what_it_was():
    """The other designs' choice (softmax over all experts, groups by their best) through the same kernel."""
    from rocml_amd import ops
    g = _gen(5)
    T, experts, top = 200, 12, 3
    z = torch.randn(T, experts, generator=g) * 2
    s = torch.softmax(z.double(), dim=-1)
    best = s.view(T, 3, 4).amax(dim=-1)
    kept = best.topk(2, dim=-1).indices
    allowed = torch.zeros(T, 3, dtype=torch.bool).scatter_(1, kept, True)[:, :, None].expand(T, 3, 4).reshape(T, experts)
    want_e = s.masked_fill(~allowed, -1.0).topk(top, dim=-1).indices
    want_w = s.gather(1, want_e)
    want_w = want_w / (want_w.sum(-1, keepdim=True) + 1e-20)
    chosen = torch.empty(T, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(T, top, dtype=torch.float32, device=DEV)
    ops.moe_route(z.to(DEV), top, (3, 2), 1e-20, chosen, weight)
    assert torch.equal(chosen.cpu().long(), want_e)
    _close(weight, want_w, 1e-5)


def test_small_sums_and_the_soft_cap():
    from rocml_amd import ops
    g = _gen(9)
    T, n = 7, 70
    x, a, b = (torch.randn(T, n, generator=g) for _ in range(3))
    gate = torch.randn(T, 3, generator=g) * 2
    xs = x.clone().to(DEV)
    ops.row_gate_add(xs, a.to(DEV), gate.to(DEV)[:, 1:2])
    _close(xs, x.double() + torch.sigmoid(gate[:, 1:2].double()) * a.double(), 1e-6, "gated row sum")
    out = x.clone().to(DEV)
    ops.weighted_sum(out, [a.to(DEV), b.to(DEV)], [0.6, -0.9], alpha=0.0)
    _close(out, 0.6 * a.double() - 0.9 * b.double(), 1e-6, "weighted sum, written")
    out = x.clone().to(DEV)
    ops.weighted_sum(out, [a.to(DEV)], [1.25], alpha=1.0)
    _close(out, x.double() + 1.25 * a.double(), 1e-6, "weighted sum, added")
    z = (torch.randn(T, n, generator=g) * 40).to(DEV)
    want = 12.0 * torch.tanh(z.cpu().double() / 12.0)
    ops.softcap(z, 12.0)
    _close(z, want, 1e-6, "soft cap")


@pytest.mark.parametrize("n", [5, 36, 70, 72, 1024, 4100])
def test_sublayer_norm_with_the_next_norm(n):
    """The kernel that norms a sublayer's output and adds it to the stream also forms the norm that reads the stream next,
    with and without the pieces of a product in place of the sublayer's output."""
    from rocml_amd import ops
    g = _gen(n)
    rows, eps, eps2 = 6, 1e-5, 1e-3
    x, y = torch.randn(rows, n, generator=g) * 3, torch.randn(rows, n, generator=g) * 5
    parts = torch.randn(2, rows, n, generator=g)
    w, w2 = 0.3 * torch.randn(n, generator=g), 0.3 * torch.randn(n, generator=g)
    for with_parts in (False, True):
        total = y.double() + (parts.double().sum(0) if with_parts else 0)
        new_x = x.double() + plain.offset_norm(total, w.double(), eps)
        want_next = plain.offset_norm(new_x, w2.double(), eps2)
        for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
            xs = x.clone().to(DEV)
            nxt = torch.empty(rows, n, dtype=dtype, device=DEV)
            ops.norm_add(xs, y.clone().to(DEV), (1 + w).to(DEV), None, eps, layer=False, copy=nxt, partials=parts.to(DEV) if with_parts else None,
                         next_gain=(1 + w2).to(DEV), next_eps=eps2)
            _close(xs, new_x, 1e-5, "stream")
            _close(nxt, want_next, tol, "the next norm")
