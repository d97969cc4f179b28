"""Each mechanism of the Sogavik layers alone, kernel against the plain functions: the layer norm and the norm of
a sublayer's output added to the stream, the stretched rotation's table, the norm of q and k over their whole
rows with biases and a partial rotation, the window's edge with one key made to stand out just inside and just
outside it (prompt and single-token kernels, at page borders), the gate per head, the matrix memory carried
through pieces and slots with gates that forget nothing and gates that forget everything, its head norm and
gate, the token-side gate, and the choice of experts by their logits with a bias."""

import pytest
import torch

from tests.plain import sogavik_plain as plain

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


@pytest.mark.parametrize("n", [1, 36, 72, 211, 1024, 4100, 8192, 8200])
def test_layer_norm_and_sublayer_norm_added_to_the_stream(n):
    from rocml_amd import ops
    g = _gen(n)
    rows = 7
    x, y = torch.randn(rows, n, generator=g) * 3, torch.randn(rows, n, generator=g) * 5 + 2.0      # a mean far from zero
    w, b = 1 + 0.3 * torch.randn(n, generator=g), 0.5 * torch.randn(n, generator=g)
    eps = 1e-3
    want_ln = plain.layer_norm(y.double(), w.double(), b.double(), eps)
    pick = torch.tensor([5, 0, 5, 2], dtype=torch.int32)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        out = torch.empty(4, n, dtype=dtype, device=DEV)
        ops.layernorm(y.to(DEV), w.to(DEV), b.to(DEV), eps, out, rows=pick.to(DEV))
        _close(out, want_ln[pick.long()], tol, "layer norm of picked rows")
    out = torch.empty(rows, n, dtype=torch.float32, device=DEV)
    ops.layernorm(y.to(DEV), w.to(DEV), b.to(DEV), eps, out)
    _close(out, want_ln, 1e-5, "layer norm")
    for layer, want in ((True, x.double() + want_ln), (False, x.double() + plain.rms(y.double(), eps) * w.double())):
        for copy_type in (None, torch.bfloat16, torch.float32):
            xs = x.clone().to(DEV)
            copy = None if copy_type is None else torch.empty(rows, n, dtype=copy_type, device=DEV)
            ops.norm_add(xs, y.to(DEV), w.to(DEV), b.to(DEV) if layer else None, eps, layer=layer, copy=copy)
            _close(xs, want, 1e-5, f"stream, layer={layer}")
            if copy is not None:
                _close(copy, want, 1e-2 if copy_type == torch.bfloat16 else 1e-5, "copy")


@pytest.mark.parametrize("n", [36, 211, 1024, 8200])
def test_sublayer_norm_adds_the_pieces_of_a_product(n):
    """The kernel is handed a product's K pieces instead of its sum: on top of what the buffer holds, or as all of it."""
    from rocml_amd import ops
    g = _gen(n + 1)
    rows, eps = 5, 1e-5
    x, y = torch.randn(rows, n, generator=g), torch.randn(rows, n, generator=g)
    parts = torch.randn(3, rows, n, generator=g) * 2
    w, b = 1 + 0.3 * torch.randn(n, generator=g), 0.5 * torch.randn(n, generator=g)
    for replace in (False, True):
        total = parts.double().sum(0) + (0 if replace else y.double())
        for layer, want in ((True, x.double() + plain.layer_norm(total, w.double(), b.double(), eps)),
                            (False, x.double() + plain.rms(total, eps) * w.double())):
            xs = x.clone().to(DEV)
            ys = (y.clone() if not replace else torch.full((rows, n), float("nan"))).to(DEV)
            copy = torch.empty(rows, n, dtype=torch.bfloat16, device=DEV)
            ops.norm_add(xs, ys, w.to(DEV), b.to(DEV) if layer else None, eps, layer=layer, copy=copy, partials=parts.to(DEV),
                         replace=replace)
            _close(xs, want, 1e-5, f"stream, layer={layer}, replace={replace}")
            _close(copy, want, 1e-2, "copy")


@pytest.mark.parametrize("n", [36, 72, 1024, 4096])
@pytest.mark.parametrize("n_branches", [1, 2])
def test_branch_norms_sublayer_norm_and_sum_in_one_kernel(n, n_branches):
    """Two mixers' outputs of very different size, each normed over the width with its own gain, half their sum, its
    norm, the residual sum and the copy."""
    from rocml_amd import ops
    g = _gen(n + n_branches)
    rows, eps_b, eps = 6, 1e-4, 1e-3
    x = torch.randn(rows, n, generator=g)
    ys = [torch.randn(rows, n, generator=g) * s + 0.5 for s in (20.0, 0.05)][:n_branches]
    gs = [1 + 0.3 * torch.randn(n, generator=g) for _ in ys]
    w, b = 1 + 0.3 * torch.randn(n, generator=g), 0.5 * torch.randn(n, generator=g)
    assert ops.norm_add_branches_fits(n, n_branches) and not ops.norm_add_branches_fits(70, 2) and not ops.norm_add_branches_fits(8192, 2)
    total = 0.5 * sum(plain.rms(y.double(), eps_b) * gg.double() for y, gg in zip(ys, gs))
    for layer, want in ((True, x.double() + plain.layer_norm(total, w.double(), b.double(), eps)),
                        (False, x.double() + plain.rms(total, eps) * w.double())):
        for copy_type in (None, torch.bfloat16, torch.float32):
            xs = x.clone().to(DEV)
            copy = None if copy_type is None else torch.empty(rows, n, dtype=copy_type, device=DEV)
            ops.norm_add_branches(xs, [y.to(DEV) for y in ys], [gg.to(DEV) for gg in gs], 0.5, eps_b, w.to(DEV),
                                  b.to(DEV) if layer else None, eps, layer=layer, copy=copy)
            _close(xs, want, 1e-5, f"stream, layer={layer}")
            if copy is not None:
                _close(copy, want, 1e-2 if copy_type == torch.bfloat16 else 1e-5, "copy")


def test_rotation_table_with_a_magnitude():
    from rocml_amd import ops
    rot = {"base": 5000.0, "dims": 12, "scaling": {"factor": 3.0, "original": 64, "fast": 8.0, "slow": 2.0}}
    f, mag = plain.rotary_frequencies(rot)
    assert mag > 1.05
    pos = torch.tensor([0, 1, 63, 64, 1000, 40000], dtype=torch.int32)
    cos = torch.empty(6, 6, dtype=torch.float32, device=DEV)
    sin = torch.empty_like(cos)
    ops.rope_table(pos.to(DEV), torch.tensor(f, dtype=D64, device=DEV), cos, sin, mag)
    ang = pos.double()[:, None] * torch.tensor(f, dtype=D64)[None, :]
    _close(cos, torch.cos(ang) * mag, 1e-6)
    _close(sin, torch.sin(ang) * mag, 1e-6)


def _prepare(q, k, v, qb, kb, vb, qg, kg, rot, dtype, positions, n_pages, perm, eps):
    """Rows of one sequence through the factors' kernel and the norm-rotation-append kernel: the norm spans a token's
    whole q row and whole k row.  Returns the prepared queries and the cache."""
    from rocml_amd import ops
    T, H, d = q.shape
    G, dv = k.shape[1], v.shape[2]
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).float().to(DEV).contiguous()
    bias = torch.cat([qb, kb, vb]).float().to(DEV)
    kc = torch.zeros((n_pages, G, PAGE, d), dtype=dtype, device=DEV)
    vc = torch.zeros((n_pages, G, dv, PAGE), dtype=dtype, device=DEV)
    table = torch.full((1, 16), -1, dtype=torch.int32)
    table[0, :len(perm)] = perm.to(torch.int32)
    table = table.to(DEV)
    q_out = torch.empty((T, H * d), dtype=dtype, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
    cos = sin = None
    dims = 0
    if rot is not None:
        f, mag = plain.rotary_frequencies(rot)
        dims = rot["dims"]
        cos = torch.empty(T, dims // 2, dtype=torch.float32, device=DEV)
        sin = torch.empty_like(cos)
        ops.rope_table(pos, torch.tensor(f, dtype=D64, device=DEV), cos, sin, mag)
    inv = torch.empty(T, 2, dtype=torch.float32, device=DEV)
    ops.qk_span_stats(qkv, H * d, G * d, bias, eps, inv)
    ops.qk_norm_rope_append(qkv, H, G, d, qg.float().to(DEV), kg.float().to(DEV), eps, cos, sin, dims, q_out, kc, vc, table, seq, pos,
                            write_kv=True, bias=bias, v_head_dim=dv, span_inv=inv)
    return q_out, kc, vc, table, seq, pos


def _plain_qk(q, k, qb, kb, qg, kg, rot, positions, eps):
    T, H, d = q.shape
    G = k.shape[1]
    qn = (plain.rms(q.reshape(T, -1).double() + qb.double(), eps) * qg.double()).reshape(T, H, d)
    kn = (plain.rms(k.reshape(T, -1).double() + kb.double(), eps) * kg.double()).reshape(T, G, d)
    if rot is not None:
        p = torch.tensor(positions)
        qn, kn = plain.rotate(qn, p, rot), plain.rotate(kn, p, rot)
    return qn, kn


@pytest.mark.parametrize("d,dv,H,G,dims,dtype,tol", [
    (40, 40, 4, 2, 12, torch.float32, 2e-5),       # a part of the head turns
    (24, 40, 3, 3, 24, torch.float32, 2e-5),       # all of it, a value head of another size
    (64, 64, 4, 1, 64, torch.bfloat16, 3e-2),      # the matrix-core kernels' sizes
    (128, 128, 2, 2, 64, torch.bfloat16, 3e-2),
    (128, 128, 4, 2, 128, torch.float32, 2e-5),    # the kernel that takes several rows a wave (prompts, whole head turned)
    (48, 16, 2, 1, 0, torch.bfloat16, 3e-2)])      # no rotation
@pytest.mark.parametrize("window,first", [(1, 0), (5, 3), (64, 0), (65, 62), (130, 0), (200, 1)])
def test_window_edges_with_a_norm_over_the_whole_projection(d, dv, H, G, dims, dtype, tol, window, first):
    """The last query points the way of the key just inside its window, and the key just outside it is the same
    vector three times as long: a window that is one too wide gives that key nearly all the weight.  The sequence
    starts at position ``first`` of its pages so that the edges fall on other places of a page."""
    from rocml_amd import ops
    T, scale, eps = 330, 10.0 / d ** 0.5, 1e-5
    g = _gen(d + window)
    rot = None if dims == 0 else {"base": 10000.0, "dims": dims, "scaling": {"factor": 2.0, "original": 64, "fast": 8.0, "slow": 1.0}}
    q, k, v = torch.randn(T, H, d, generator=g), torch.randn(T, G, d, generator=g), torch.randn(T, G, dv, generator=g)
    qb, kb, vb = 0.3 * torch.randn(H * d, generator=g), 0.3 * torch.randn(G * d, generator=g), 0.3 * torch.randn(G * dv, generator=g)
    qg, kg = 1 + 0.3 * torch.randn(H * d, generator=g), 1 + 0.3 * torch.randn(G * d, generator=g)
    positions = list(range(first, first + T))
    n_pages = (first + T) // PAGE + 3
    perm = torch.randperm(n_pages, generator=g)[:(first + T + PAGE - 1) // PAGE]
    q_out, kc, vc, table, seq, pos = _prepare(q, k, v, qb, kb, vb, qg, kg, rot, dtype, positions, n_pages, perm, eps)
    qn, kn = _plain_qk(q, k, qb, kb, qg, kg, rot, positions, eps)
    _close(q_out.reshape(T, H, d), qn, 1e-5 if dtype == torch.float32 else 1e-2, "prepared queries")
    # the plain functions take keys as they are: plant the two keys in the cache itself, and in the plain keys
    inside, outside = T - window, T - window - 1
    rep = H // G
    for a in range(G):
        target = qn[T - 1, a * rep] / qn[T - 1, a * rep].norm() * d ** 0.5
        for j, length in ((inside, 1.0), (outside, 3.0)):
            if j < 0:
                continue
            kn[j, a] = target * length
            p = first + j
            kc[int(perm[p // PAGE]), a, p % PAGE] = (target * length).to(dtype).to(DEV)
    # (in bfloat16 the kernels are handed queries, keys and values rounded to it: the plain function gets the same)
    def seen(t):
        return t.to(dtype).double() if dtype != torch.float32 else t
    want = plain.attend(seen(qn), seen(kn), seen((v.reshape(T, -1).double() + vb.double()).reshape(T, G, dv)), scale, window)
    if outside >= 0 and window > 1:
        s = (qn[T - 1, 0] @ kn[:, 0].T) * scale
        assert s[outside] > s[inside] + 5, "the key outside the window would win if it were seen"
    out = torch.empty((T, H * dv), dtype=dtype, device=DEV)
    cu = torch.tensor([0, T], dtype=torch.int32, device=DEV)
    scratch = torch.empty(64 << 20, dtype=torch.uint8, device=DEV)
    ops.attention(q_out, out, kc, vc, table, seq, pos, H, G, d, scale, window, workspace=scratch, cu_seqlens=cu, max_new=T,
                  q_counts=(T,), max_len=first + T, v_head_dim=dv)
    _close(out.reshape(T, H, dv)[T - 1], want[T - 1], tol, "prompt kernel, last query")
    # (the pages hold nothing at the positions before ``first``, which the plain function does not know of: the
    # queries whose windows reach back there are left out)
    whole = 0 if first == 0 else window - 1
    _close(out.reshape(T, H, dv)[whole:], want[whole:], tol, "prompt kernel")
    one = torch.empty((1, H * dv), dtype=dtype, device=DEV)
    ops.attention(q_out[T - 1:].contiguous(), one, kc, vc, table, seq[:1], pos[T - 1:].contiguous(), H, G, d, scale, window,
                  workspace=scratch, cu_seqlens=torch.tensor([0, 1], dtype=torch.int32, device=DEV), max_new=1, q_counts=(1,),
                  max_len=first + T, n_splits=ops.decode_splits(G, 256, 16), v_head_dim=dv)
    _close(one.reshape(H, dv), want[T - 1], tol, "single-token kernel")


@pytest.mark.parametrize("d,dv,H,G,dims", [(40, 40, 4, 2, 12), (24, 40, 3, 3, 24), (128, 128, 4, 2, 128), (64, 64, 16, 1, 0), (10, 6, 1, 1, 2)])
def test_whole_row_norm_formed_inside_the_kernel(d, dv, H, G, dims):
    """A step of few tokens has no kernel of its own for the norm's factors: queries and the keys in the cache must
    come out as with it."""
    from rocml_amd import ops
    T, eps = 9, 1e-4
    g = _gen(d * 7 + H)
    rot = None if dims == 0 else {"base": 10000.0, "dims": dims}
    q, k, v = torch.randn(T, H, d, generator=g) * 3, torch.randn(T, G, d, generator=g) * 0.2, torch.randn(T, G, dv, generator=g)
    qb, kb, vb = 0.3 * torch.randn(H * d, generator=g), 0.3 * torch.randn(G * d, generator=g), 0.3 * torch.randn(G * dv, generator=g)
    qg, kg = 1 + 0.3 * torch.randn(H * d, generator=g), 1 + 0.3 * torch.randn(G * d, generator=g)
    positions = list(range(60, 60 + T))                     # across a page's border
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).float().to(DEV).contiguous()
    bias = torch.cat([qb, kb, vb]).float().to(DEV)
    kc = torch.zeros((4, G, PAGE, d), dtype=torch.float32, device=DEV)
    vc = torch.zeros((4, G, dv, PAGE), dtype=torch.float32, device=DEV)
    table = torch.tensor([[2, 0, -1, -1]], dtype=torch.int32, device=DEV)
    q_out = torch.empty((T, H * d), dtype=torch.float32, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
    cos = sin = None
    if rot is not None:
        f, mag = plain.rotary_frequencies(rot)
        cos = torch.empty(T, dims // 2, dtype=torch.float32, device=DEV)
        sin = torch.empty_like(cos)
        ops.rope_table(pos, torch.tensor(f, dtype=D64, device=DEV), cos, sin, mag)
    ops.qk_norm_rope_append(qkv, H, G, d, qg.to(DEV), kg.to(DEV), eps, cos, sin, dims, q_out, kc, vc, table, seq, pos,
                            write_kv=True, bias=bias, v_head_dim=dv, span_self=True)
    qn, kn = _plain_qk(q, k, qb, kb, qg, kg, rot, positions, eps)
    _close(q_out.reshape(T, H, d), qn, 1e-5, "queries")
    for j, p in enumerate(positions):
        page = 2 if p < PAGE else 0
        _close(kc[page, :, p % PAGE], kn[j], 1e-5, f"key at {p}")
        _close(vc[page, :, :, p % PAGE], (v[j].reshape(-1).double() + vb.double()).reshape(G, dv), 1e-6, f"value at {p}")


def test_gate_per_head():
    from rocml_amd import ops
    g = _gen(5)
    H, dv = 5, 24
    y, gate = torch.randn(9, H * dv, generator=g), torch.randn(9, 100, generator=g) * 3
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2)):
        out = y.to(dtype).to(DEV)
        ops.sigmoid_gate(out, gate.to(DEV)[:, 95:], group=dv)
        want = y.to(dtype).double().reshape(9, H, dv) * torch.sigmoid(gate[:, 95:].double())[:, :, None]
        _close(out, want.reshape(9, -1), tol)
    one = y[:1].contiguous().to(DEV)          # a single row, as a step of one token has it
    ops.sigmoid_gate(one, gate.to(DEV)[:1, 95:], group=dv)
    _close(one, (y[:1].double().reshape(1, H, dv) * torch.sigmoid(gate[:1, 95:].double())[:, :, None]).reshape(1, -1), 1e-6)


def _pieces(total, sizes):
    out, at = [], 0
    for n in sizes:
        if at >= total:
            break
        out.append((at, min(total, at + n)))
        at += n
    if at < total:
        out.append((at, total))
    return out


def _memory_run(proj, cols, ib, fb, cap, H, dk, dv, lengths, pieces, slots, n_slots):
    """The matrix memory over several sequences (rows of ``proj`` one sequence after the other), every sequence cut
    into the same pieces, each piece one launch for all sequences that still have tokens."""
    from rocml_amd import ops
    tiles = ops.mlstm_tiles(dv)
    S = torch.full((n_slots, H, dv, dk), 7.0, device=DEV)         # slots of other sequences hold something else
    N = torch.full((n_slots, H, tiles, dk), -3.0, device=DEV)
    M = torch.full((n_slots, H, tiles), 2.0, device=DEV)
    for s in slots:
        S[s].zero_(); N[s].zero_(); M[s].zero_()
    starts = [sum(lengths[:i]) for i in range(len(lengths))]
    out = torch.zeros(sum(lengths), H * dv, dtype=torch.float32)
    for lo, hi in _pieces(max(lengths), pieces):
        live = [i for i, n in enumerate(lengths) if n > lo]
        rows = [list(range(starts[i] + lo, starts[i] + min(hi, lengths[i]))) for i in live]
        flat = [r for rr in rows for r in rr]
        cu = torch.tensor([0] + list(torch.tensor([len(r) for r in rows]).cumsum(0)), dtype=torch.int32, device=DEV)
        part = proj[flat].contiguous().to(DEV)
        o = torch.empty(len(flat), H * dv, dtype=torch.float32, device=DEV)
        ops.mlstm_scan(part, *cols, ib.to(DEV), fb.to(DEV), cap, dk ** -0.5, 1e-6, S, N, M, cu,
                       torch.tensor([slots[i] for i in live], dtype=torch.int32, device=DEV), o, H, dk, dv)
        out[flat] = o.cpu()
    others = [s for s in range(n_slots) if s not in slots]
    if others:
        assert float((S[others] - 7.0).abs().max()) == 0.0 and float((M[others] - 2.0).abs().max()) == 0.0, "other slots were touched"
    return out


def _memory_plain(proj, cols, ib, fb, cap, H, dk, dv, lengths):
    q0, k0, v0, i0, f0 = cols
    out, at = [], 0
    p = proj.double()
    for n in lengths:
        r = p[at:at + n]
        q = r[:, q0:q0 + H * dk].reshape(n, H, dk) * dk ** -0.5
        k = r[:, k0:k0 + H * dk].reshape(n, H, dk)
        v = r[:, v0:v0 + H * dv].reshape(n, H, dv)
        ig = cap * torch.tanh((r[:, i0:i0 + H] + ib.double()) / cap)
        fg = plain.log_sigmoid(cap * torch.tanh((r[:, f0:f0 + H] + fb.double()) / cap))
        out.append(plain.matrix_memory_scan(q, k, v, ig, fg).reshape(n, H * dv))
        at += n
    return torch.cat(out)


@pytest.mark.parametrize("H,dk,dv", [(2, 20, 36), (3, 17, 9), (1, 1, 12), (4, 6, 1), (2, 64, 64), (1, 128, 32), (1, 200, 40), (2, 96, 100)])
@pytest.mark.parametrize("pieces", [[1000], [1, 1, 2, 31, 32, 33, 1], [2] * 40, [64, 7]])
def test_matrix_memory_carried_through_pieces(H, dk, dv, pieces):
    g = _gen(dk * 100 + dv)
    lengths = [70, 1, 33]
    T = sum(lengths)
    lead = 3                                    # the mixer's columns do not start at the row's first number
    width = lead + 2 * H * dk + H * dv + 2 * H + 5
    proj = torch.randn(T, width, generator=g)
    cols = (lead, lead + H * dk, lead + 2 * H * dk, lead + 2 * H * dk + H * dv + 1, lead + 2 * H * dk + H * dv + 1 + H)
    proj[:, cols[3]:cols[3] + H] *= 3.0        # input gates from -3 to 3 sigma
    proj[:, cols[4]:cols[4] + H] = proj[:, cols[4]:cols[4] + H] * 2.0 + 1.0
    ib, fb = torch.randn(H, generator=g), torch.randn(H, generator=g)
    got = _memory_run(proj, cols, ib, fb, 5.0, H, dk, dv, lengths, pieces, slots=[4, 0, 2], n_slots=6)
    _close(got, _memory_plain(proj, cols, ib, fb, 5.0, H, dk, dv, lengths), 2e-5)


@pytest.mark.parametrize("forget,take", [(30.0, -30.0), (30.0, 30.0), (-30.0, 30.0), (-30.0, -30.0), (0.0, 0.0)])
def test_matrix_memory_gates_at_their_limits(forget, take):
    """A forget gate of one keeps the first token's pair for 300 tokens (a query along that key finds its value), one
    of nearly zero drops it at once; input gates at the cap on either side; the running maximum starts at zero, so
    small input gates are not scaled up."""
    g = _gen(int(forget + 2 * take) + 100)
    H, dk, dv, T, cap = 2, 24, 40, 300, 20.0
    cols = (0, H * dk, 2 * H * dk, 2 * H * dk + H * dv, 2 * H * dk + H * dv + H)
    proj = torch.randn(T, cols[4] + H, generator=g)
    # (queries and keys of one sign: n . q is then a sum without cancellation, and what is compared is the
    # recurrence, not the rounding of a denominator that happens to come out near zero)
    proj[:, :cols[2]] = proj[:, :cols[2]].abs()
    proj[:, cols[3]:cols[3] + H] = take + 0.1 * proj[:, cols[3]:cols[3] + H]
    proj[:, cols[4]:cols[4] + H] = forget + 0.1 * proj[:, cols[4]:cols[4] + H]
    proj[T - 1, cols[0]:cols[0] + H * dk] = proj[0, cols[1]:cols[1] + H * dk] * 4.0      # the last query along the first key
    zero = torch.zeros(H)
    want = _memory_plain(proj, cols, zero, zero, cap, H, dk, dv, [T])
    for pieces in ([1000], [1] * 300, [299, 1]):
        got = _memory_run(proj, cols, zero, zero, cap, H, dk, dv, [T], pieces, slots=[1], n_slots=2)
        _close(got, want, 3e-5, f"pieces {pieces[:3]}")
        assert torch.isfinite(got).all()


@pytest.mark.parametrize("H,dv,dtype,tol", [(2, 36, torch.float32, 1e-5), (3, 9, torch.float32, 1e-5), (4, 1, torch.float32, 1e-5),
                                            (4, 128, torch.bfloat16, 1e-2), (1, 200, torch.bfloat16, 1e-2)])
def test_head_norm_and_gate(H, dv, dtype, tol):
    from rocml_amd import ops
    g = _gen(H * dv)
    T, lead, eps = 11, 7, 1e-4
    o = torch.randn(T, H * dv, generator=g) * torch.rand(T, 1, generator=g) * 10
    z = torch.randn(T, lead + H * dv + 2, generator=g) * 2
    w = 1 + 0.3 * torch.randn(H * dv, generator=g)
    out = torch.empty(T, H * dv, dtype=dtype, device=DEV)
    ops.head_norm_gate(o.to(DEV), z.to(DEV), lead, w.to(DEV), out, H, eps)
    want = plain.rms(o.double().reshape(T, H, dv), eps).reshape(T, -1) * w.double() * torch.sigmoid(z[:, lead:lead + H * dv].double())
    _close(out, want, tol)


@pytest.mark.parametrize("dim,col0,cols", [(5, 10, 20), (1, 3, 4), (16, 0, 16), (64, 64, 192)])
def test_token_side_gate(dim, col0, cols):
    from rocml_amd import ops
    g = _gen(dim)
    T, vocab = 13, 50
    z = torch.randn(T, dim, generator=g) * 2
    ids = torch.randint(0, vocab, (T,), generator=g).to(torch.int32)
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2)):
        table = torch.randn(vocab, cols, generator=g).to(dtype)
        out = torch.empty(T, dim, dtype=dtype, device=DEV)
        ops.token_side_gate(z.to(DEV), table.to(DEV), ids.to(DEV), col0, out)
        _close(out, plain.gelu_tanh(z.double()) * table.double()[ids.long()][:, col0:col0 + dim], tol)


@pytest.mark.parametrize("E,top", [(6, 2), (5, 1), (3, 3), (1, 1), (16, 4), (130, 7)])
def test_experts_chosen_by_logit_weighted_by_the_softmax_over_the_chosen(E, top):
    from rocml_amd import ops
    ops.prepare(("moe",))
    g = _gen(E)
    T = 40
    logits = torch.randn(T, E, generator=g) * 4
    logits[0] = logits[0] - 60.0               # far below zero: the softmax over all experts would lose nothing either
    logits[1, 0] = 50.0                        # one expert far above the others: the others' weights are tiny, not zero
    bias = torch.randn(E, generator=g)
    z = logits.clone().to(DEV)
    chosen = torch.empty(T, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(T, top, dtype=torch.float32, device=DEV)
    ops.moe_route(z, top, None, 0.0, chosen, weight, bias=bias.to(DEV))
    want_c, want_w = plain.choose(logits.double() + bias.double(), top)
    order = torch.argsort(chosen.cpu().long(), dim=1)
    want_order = torch.argsort(want_c, dim=1)
    assert torch.equal(torch.gather(chosen.cpu().long(), 1, order), torch.gather(want_c, 1, want_order))
    _close(torch.gather(weight.cpu(), 1, order), torch.gather(want_w, 1, want_order), 1e-5)
