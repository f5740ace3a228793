"""Each mechanism of the Felovik layers alone, kernel against the plain functions: the embedding with
learned positions, the query's stretch at the positions where it changes, the attention with one key
made to stand out far away and at page borders (prompt and single-token kernels), the output gate,
the causal convolution and the recurrence carried through pieces, slots used again, decays close to
one and to zero, the gated norm in parts, the limited gated activation, the experts' choice with and
without groups, the experts' products on both kinds of kernel, and the sum with its norm."""

import pytest
import torch

from tests.plain import felovik_plain as plain

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


def test_embedding_adds_the_row_of_the_position():
    from rocml_amd import ops
    g = _gen(1)
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-6)):
        table = torch.randn(50, 24, generator=g).to(dtype)
        pos_table = torch.randn(40, 24, generator=g).to(dtype)
        ids = torch.tensor([3, 49, 0, 7, 7], dtype=torch.int32)
        out = torch.empty(5, 24, dtype=torch.float32, device=DEV)
        ops.embed_gather(table.to(DEV), ids.to(DEV), out, 2.5, pos_table=pos_table.to(DEV),
                         positions=torch.tensor([10, 11, 12, 0, 39], dtype=torch.int32, device=DEV))
        want = plain.embed({"embed": table.double(), "pos": pos_table.double()}, ids.tolist(), 2.5, first=10)
        _close(out[:3], want[:3], tol)
        _close(out[3], table[7].double() * 2.5 + pos_table[0].double(), tol)
        _close(out[4], table[7].double() * 2.5 + pos_table[39].double(), tol)


def _qkv_step(q, k, v, dtype, positions, n_pages, perm, q_temp, eps):
    """Queries, keys and values of one sequence (rows are positions) through the norm-and-append kernel:
    returns the prepared queries and the cache."""
    from rocml_amd import ops
    T, H, d = q.shape
    G, dv = k.shape[1], v.shape[2]
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).float().to(DEV).contiguous()
    kc = torch.zeros((n_pages, G, PAGE, d), dtype=dtype, device=DEV)
    vc = torch.zeros((n_pages, G, dv, PAGE), dtype=dtype, device=DEV)
    table = torch.full((1, 16), -1, dtype=torch.int32)
    table[0, :len(perm)] = perm.to(torch.int32)
    table = table.to(DEV)
    ones = torch.ones(d, dtype=torch.float32, device=DEV)
    q_out = torch.empty((T, H * d), dtype=dtype, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
    ops.qk_norm_rope_append(qkv, H, G, d, ones, ones, eps, None, None, 0, q_out, kc, vc, table, seq, pos, write_kv=True,
                            v_head_dim=dv, q_temp=q_temp)
    return q_out, kc, vc, table, seq, pos


@pytest.mark.parametrize("d,dv,H,G,dtype,tol", [(40, 40, 4, 2, torch.float32, 2e-5), (24, 40, 3, 3, torch.float32, 2e-5),
                                                (64, 64, 4, 1, torch.bfloat16, 3e-2), (128, 128, 2, 2, torch.bfloat16, 3e-2),
                                                (48, 16, 2, 1, torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("far", [0, 63, 64, 127, 128, 448, 637])
def test_attention_finds_one_key_far_away(d, dv, H, G, dtype, tol, far):
    """The last query and one key at ``far`` point the same way, so that key's weight is close to one; the
    stretch changes at positions 99, 199, ... (every 100).  The prompt kernel sees all 640 positions, the
    single-token kernel only the last query."""
    from rocml_amd import ops
    T, scale, eps, q_temp = 640, 10.0 / d, 1e-5, (0.6, 100)
    g = _gen(d + far)
    q, k, v = torch.randn(T, H, d, generator=g), torch.randn(T, G, d, generator=g), torch.randn(T, G, dv, generator=g)
    rep = H // G
    for a in range(H):
        q[T - 1, a] = k[far, a // rep] * 3.0        # (the norm takes the length away)
    n_pages = T // PAGE + 3
    perm = torch.randperm(n_pages, generator=g)[:T // PAGE]
    q_out, kc, vc, table, seq, pos = _qkv_step(q, k, v, dtype, list(range(T)), n_pages, perm, q_temp, eps)
    qn, kn = plain.rms(q.double(), eps), plain.rms(k.double(), eps)
    temp = plain.query_temperature(torch.arange(T), *q_temp)
    want = plain.attend(qn * temp[:, None, None], kn, v.double(), scale)
    weight_far = torch.softmax((qn[T - 1, 0] * temp[T - 1]) @ kn[:, 0].T * scale, dim=-1)[far]
    assert weight_far > 0.9, "the test's key does not stand out"
    _close(q_out.reshape(T, H, d), qn * temp[:, None, None], 1e-5 if dtype == torch.float32 else 1e-2, "prepared queries")
    out = torch.empty((T, H * dv), dtype=dtype, device=DEV)
    cu = torch.tensor([0, T], dtype=torch.int32, device=DEV)
    scratch = torch.empty(64 << 20, dtype=torch.uint8, device=DEV)
    ops.attention(q_out, out, kc, vc, table, seq, pos, H, G, d, scale, None, workspace=scratch, cu_seqlens=cu, max_new=T,
                  q_counts=(T,), max_len=T, v_head_dim=dv)
    _close(out.reshape(T, H, dv), want, tol, "prompt kernel")
    one = torch.empty((1, H * dv), dtype=dtype, device=DEV)
    ops.attention(q_out[T - 1:].contiguous(), one, kc, vc, table, seq[:1], pos[T - 1:].contiguous(), H, G, d, scale, None,
                  workspace=scratch, cu_seqlens=torch.tensor([0, 1], dtype=torch.int32, device=DEV), max_new=1, q_counts=(1,),
                  max_len=T, n_splits=ops.decode_splits(G, 256, 16), v_head_dim=dv)
    _close(one.reshape(H, dv), want[T - 1], tol, "single-token kernel")


@pytest.mark.parametrize("d,T", [(128, 200), (40, 7), (64, 130)])
def test_query_stretch_changes_where_it_should(d, T):
    """Positions around the multiples of ``every``: the stretch of position ``p`` uses ``floor((p + 1) / every)``."""
    every, coef = 9, 1.25
    g = _gen(d)
    q, k, v = torch.randn(T, 2, d, generator=g), torch.randn(T, 1, d, generator=g), torch.randn(T, 1, d, generator=g)
    positions = list(range(3, 3 + T))
    q_out, *_ = _qkv_step(q, k, v, torch.float32, positions, 8, torch.arange(5), (coef, every), 1e-6)
    temp = plain.query_temperature(torch.tensor(positions), coef, every)
    assert temp[4] == temp[0] and temp[5] > temp[4], "position 8 is the first of the second step"
    _close(q_out.reshape(T, 2, d), plain.rms(q.double(), 1e-6) * temp[:, None, None], 1e-5)


def test_output_gate():
    from rocml_amd import ops
    g = _gen(5)
    y, gate = torch.randn(9, 40, generator=g), torch.randn(9, 100, generator=g) * 3
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2)):
        out = y.to(dtype).to(DEV)
        ops.sigmoid_gate(out, gate.to(DEV)[:, 60:])
        _close(out, y.to(dtype).double() * torch.sigmoid(gate[:, 60:].double()), tol)


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


@pytest.mark.parametrize("C,lead", [(37, 11), (40, 12)])
@pytest.mark.parametrize("taps", [1, 2, 4, 8])
def test_convolution_carried_through_pieces(taps, C, lead):
    """Two sequences in slots 5 and 2 of 7, fed in pieces of unequal sizes (some shorter than the taps);
    then slot 5 again from zero for a third sequence."""
    from rocml_amd import ops
    # (37 channels behind 11 others in rows of 51: one channel a thread; 40 behind 12 in rows of 56: four)
    tail = 3 if C % 4 else 4
    g = _gen(taps)
    w, b = torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    seqs = [torch.randn(n, lead + C + tail, generator=g) for n in (50, 23)]
    state = torch.zeros((7, taps - 1, C), dtype=torch.float32, device=DEV)
    state[1].fill_(9.0)                 # another sequence's memory must not leak in
    slots = [5, 2]
    plans = [_pieces(50, [1, 2, 1, 7, 3, 30]), _pieces(23, [2, 1, 1, 5])]
    got = [[], []]
    for step in range(max(len(p) for p in plans)):
        live = [i for i in range(2) if step < len(plans[i])]
        rows = [seqs[i][plans[i][step][0]:plans[i][step][1]] for i in live]
        counts = [r.shape[0] for r in rows]
        u = torch.cat(rows).to(DEV).contiguous()
        cu = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32, device=DEV)
        seq = torch.repeat_interleave(torch.arange(len(live), dtype=torch.int32), torch.tensor(counts)).to(DEV)
        out = torch.empty((sum(counts), C), dtype=torch.float32, device=DEV)
        ops.causal_conv(u, lead, C, w.t().contiguous().to(DEV), b.to(DEV), state, seq, cu, torch.tensor([slots[i] for i in live], dtype=torch.int32, device=DEV),
                        out, silu=True)
        at = 0
        for i, n in zip(live, counts):
            got[i].append(out[at:at + n].cpu())
            at += n
    for i in range(2):
        want = plain.silu(plain.causal_conv(seqs[i][:, lead:lead + C].double(), w.double(), b.double()))
        _close(torch.cat(got[i]), want, 1e-5, f"sequence {i}")
    assert taps == 1 or float(state[1].min()) == 9.0
    # the slot is handed out again: the cache zeroes it, and a new sequence starts from nothing
    state[5].zero_()
    third = torch.randn(6, lead + C + tail, generator=g)
    out = torch.empty((6, C), dtype=torch.float32, device=DEV)
    ops.causal_conv(third.to(DEV), lead, C, w.t().contiguous().to(DEV), b.to(DEV), state, torch.zeros(6, dtype=torch.int32, device=DEV),
                    torch.tensor([0, 6], dtype=torch.int32, device=DEV), torch.tensor([5], dtype=torch.int32, device=DEV), out)
    _close(out, plain.silu(plain.causal_conv(third[:, lead:lead + C].double(), w.double(), b.double())), 1e-5)


@pytest.mark.parametrize("H,P,N,G", [(4, 12, 20, 2), (2, 64, 128, 1), (3, 5, 1, 3), (6, 40, 56, 3), (2, 33, 256, 2), (1, 16, 100, 1)])
def test_recurrence_carried_through_pieces(H, P, N, G):
    """Heads whose decay is close to one (a far token still counts), close to zero, and in between; two
    sequences fed in pieces down to one token, in slots of their own."""
    from rocml_amd import ops
    g = _gen(H * 1000 + N)
    inner, bc = H * P, G * N
    a_log = torch.tensor([-6.0, 2.0, 0.0, -1.0, 1.0, -3.0][:H])
    dt_bias, d_skip = torch.randn(H, generator=g), torch.randn(H, generator=g)
    lens = (150, 40)
    xbc = [torch.randn(n, inner + 2 * bc, generator=g) for n in lens]
    dts = [torch.randn(n, 3 + H, generator=g) for n in lens]
    state = torch.zeros((4, H, P, N), dtype=torch.float32, device=DEV)
    slots = [3, 0]
    plans = [_pieces(150, [1, 1, 33, 2, 64, 40]), _pieces(40, [7, 1, 1])]
    got = [[], []]
    for step in range(max(len(p) for p in plans)):
        live = [i for i in range(2) if step < len(plans[i])]
        counts = [plans[i][step][1] - plans[i][step][0] for i in live]
        x = torch.cat([xbc[i][plans[i][step][0]:plans[i][step][1]] for i in live]).to(DEV).contiguous()
        dt = torch.cat([dts[i][plans[i][step][0]:plans[i][step][1]] for i in live]).to(DEV).contiguous()
        cu = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32, device=DEV)
        y = torch.empty((sum(counts), inner), dtype=torch.float32, device=DEV)
        ops.ssd_scan(x, dt, 3, dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV), state, cu,
                     torch.tensor([slots[i] for i in live], dtype=torch.int32, device=DEV), y, H, P, N, G)
        at = 0
        for i, n in zip(live, counts):
            got[i].append(y[at:at + n].cpu())
            at += n
    for i, n in enumerate(lens):
        v = xbc[i].double()
        want = plain.recurrence(v[:, :inner].reshape(n, H, P), v[:, inner:inner + bc].reshape(n, G, N),
                                v[:, inner + bc:].reshape(n, G, N), dts[i][:, 3:].double(), dt_bias.double(), a_log.double(),
                                d_skip.double())
        _close(torch.cat(got[i]), want.reshape(n, inner), 2e-5, f"sequence {i}")
    assert float(state[1].abs().max()) == 0.0 and float(state[2].abs().max()) == 0.0


def test_far_token_through_a_slow_decay():
    """One head that forgets almost nothing: the first token's input is large, everything after it is
    small, and the output 300 tokens later is mostly the first token's."""
    from rocml_amd import ops
    H, P, N, T = 1, 8, 16, 301
    g = _gen(9)
    x, B, C = torch.randn(T, H * P, generator=g) * 0.01, torch.randn(T, N, generator=g), torch.randn(T, N, generator=g)
    x[0] = torch.randn(P, generator=g) * 50
    C[T - 1] = B[0]
    xbc = torch.cat([x, B, C], dim=1)
    dt = torch.zeros(T, 1)
    a_log, dt_bias, d_skip = torch.tensor([-9.0]), torch.tensor([0.3]), torch.tensor([0.0])
    want = plain.recurrence(x.double().reshape(T, 1, P), B.double().reshape(T, 1, N), C.double().reshape(T, 1, N), dt.double(),
                            dt_bias.double(), a_log.double(), d_skip.double()).reshape(T, P)
    first_only = plain.softplus(torch.tensor(0.3, dtype=D64)) * float(B[0].double() @ B[0].double()) * x[0].double()
    assert float((want[T - 1] - first_only).abs().max() / want[T - 1].abs().max()) < 0.2, "the test's first token does not dominate"
    state = torch.zeros((1, H, P, N), dtype=torch.float32, device=DEV)
    y = torch.empty((T, P), dtype=torch.float32, device=DEV)
    head = 200                  # a prompt of 200, then token by token
    slot = torch.zeros(1, dtype=torch.int32, device=DEV)
    ops.ssd_scan(xbc[:head].to(DEV).contiguous(), dt[:head].to(DEV).contiguous(), 0, dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV),
                 state, torch.tensor([0, head], dtype=torch.int32, device=DEV), slot, y[:head], H, P, N, 1)
    for t in range(head, T):
        ops.ssd_scan(xbc[t:t + 1].to(DEV).contiguous(), dt[t:t + 1].to(DEV).contiguous(), 0, dt_bias.to(DEV), a_log.to(DEV),
                     d_skip.to(DEV), state, torch.tensor([0, 1], dtype=torch.int32, device=DEV), slot, y[t:t + 1], H, P, N, 1)
    _close(y, want, 2e-5)


@pytest.mark.parametrize("n,parts", [(48, 2), (36, 36), (1024, 1), (600, 3), (4096, 8), (4096, 1), (90, 5)])
def test_gated_norm_in_parts(n, parts):
    from rocml_amd import ops
    g = _gen(n)
    lead = 7 if n % 8 else 8            # (a gate that starts on a multiple of 4 numbers takes the vector kernel)
    y, z, w = torch.randn(5, n, generator=g), torch.randn(5, lead + n + (0 if n % 8 else 4), generator=g) * 2, torch.randn(n, generator=g)
    y[:, :n // parts] *= 30         # one part far larger than the others: a norm over the whole row would show
    want = plain.gated_part_norm(y.double(), z[:, lead:lead + n].double(), w.double(), parts, 1e-4)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        out = torch.empty((5, n), dtype=dtype, device=DEV)
        ops.gated_part_norm(y.to(DEV), z.to(DEV), lead, w.to(DEV), out, parts, 1e-4)
        _close(out, want, tol)


@pytest.mark.parametrize("limit", [None, 0.7, 50.0])
def test_limited_gated_activation(limit):
    from rocml_amd import ops
    g = _gen(3)
    gate, up = torch.randn(6, 30, generator=g) * 2, torch.randn(6, 30, generator=g) * 2
    want = plain.limited_gate(gate.double(), up.double(), limit)
    both = torch.stack([gate, up], dim=2).reshape(6, 60).to(DEV)
    out = torch.empty((6, 30), dtype=torch.float32, device=DEV)
    ops.swiglu(both, out, interleaved=True, activation="sigmoid_1702", limit=limit, up_offset=1.0)
    _close(out, want, 1e-6)


@pytest.mark.parametrize("E,top,groups", [(12, 4, (4, 2)), (6, 2, None), (5, 1, None), (4, 4, (2, 2)), (300, 8, (10, 3)),
                                           (64, 6, (8, 4)), (16, 4, (2, 1)), (2, 2, (1, 1))])
def test_choice_of_experts(E, top, groups):
    from rocml_amd import ops
    g = _gen(E)
    logits = torch.randn(70, E, generator=g) * 2
    r = {"experts": E, "top": top}
    if groups is not None:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    want_e, want_w = plain.choose(logits.double(), r)
    chosen = torch.empty((70, top), dtype=torch.int32, device=DEV)
    weight = torch.empty((70, top), dtype=torch.float32, device=DEV)
    ops.moe_route(logits.to(DEV), top, groups, 1e-20, chosen, weight)
    assert torch.equal(chosen.cpu().long(), want_e), "other experts (the best first)"
    _close(weight, want_w, 1e-5)
    if groups is not None and groups[1] < groups[0]:
        free_e, _ = plain.choose(logits.double(), {"experts": E, "top": top})
        assert not torch.equal(free_e, want_e), "the groups change nothing in this test"


@pytest.mark.parametrize("T,w,ff,E,top,dtype,tol", [(200, 40, 24, 3, 2, torch.float32, 2e-5), (1, 72, 40, 6, 2, torch.float32, 2e-5),
                                                    (200, 64, 48, 3, 2, torch.bfloat16, 2e-2), (5, 128, 64, 16, 4, torch.bfloat16, 2e-2),
                                                    (130, 36, 20, 4, 3, torch.bfloat16, 2e-2), (70, 64, 32, 5, 5, torch.bfloat16, 2e-2)])
def test_experts_products_and_weighted_sum(T, w, ff, E, top, dtype, tol):
    """More rows per expert than a tile holds, a single token, widths the matrix cores take and widths
    they refuse; the sum of a token's experts against the plain loop."""
    from rocml_amd import ops
    g = _gen(T + E)
    t = {"router": torch.randn(E, w, generator=g)}
    for e in range(E):
        t[f"e{e}.gate"] = (torch.randn(ff, w, generator=g) / w ** 0.5).to(dtype).float()
        t[f"e{e}.up"] = (torch.randn(ff, w, generator=g) / w ** 0.5).to(dtype).float()
        t[f"e{e}.down"] = (torch.randn(w, ff, generator=g) / ff ** 0.5).to(dtype).float()
    h = torch.randn(T, w, generator=g).to(dtype).float()
    m = {"router": {"experts": E, "top": top}}
    want = plain.routed_ff(h.double(), {k: v.double() for k, v in t.items()}, "", m)
    logits = (h.double() @ t["router"].double().T).float()
    chosen = torch.empty((T, top), dtype=torch.int32, device=DEV)
    weight = torch.empty((T, top), dtype=torch.float32, device=DEV)
    ops.moe_route(logits.to(DEV), top, None, 1e-20, chosen, weight)
    pairs = T * top
    plan = ops.moe_plan(chosen, E, torch.empty(ops.moe_plan_words(pairs, E), dtype=torch.int32, device=DEV))
    offsets, order, place = plan[0].cpu(), plan[1].cpu(), plan[2].cpu()
    assert int(offsets[-1]) == pairs and sorted(order.tolist()) == list(range(pairs))
    assert all(int(place[int(p)]) == i for i, p in enumerate(order))
    flat = chosen.cpu().reshape(-1)
    assert all(int(offsets[int(flat[int(p)])]) <= i < int(offsets[int(flat[int(p)]) + 1]) for i, p in enumerate(order))
    stack = lambda kind: torch.stack([t[f"e{e}.{kind}"] for e in range(E)]).to(dtype).to(DEV).contiguous()
    hid = torch.empty((pairs, ff), dtype=dtype, device=DEV)
    ops.moe_gemm(h.to(dtype).to(DEV), stack("gate"), hid, plan, top, gather=True, w2=stack("up"))
    y = torch.empty((pairs, w), dtype=torch.float32, device=DEV)
    ops.moe_gemm(hid, stack("down"), y, plan, top, gather=False)
    out = torch.full((T, w), float("nan"), dtype=torch.float32, device=DEV)
    ops.moe_combine(y, plan, weight, out)
    _close(out, want, tol)
    base = torch.randn(T, w, generator=g)
    acc = base.to(DEV)
    ops.moe_combine(y, plan, weight, acc, accumulate=True)
    _close(acc, want + base.double(), tol)
    if dtype == torch.bfloat16 and w % 8 == 0 and ff % 8 == 0:
        # the matrix-core kernel against the plain one on the same operands
        hid2 = torch.empty_like(hid)
        ops.moe_gemm(h.to(dtype).to(DEV), stack("gate"), hid2, plan, top, gather=True, w2=stack("up"), plain=True)
        _close(hid, hid2.double().cpu(), 2e-2)


@pytest.mark.parametrize("n", [72, 70, 2048, 9000])
def test_sum_and_norm(n):
    from rocml_amd import ops
    g = _gen(12)
    T, eps = 9, 1e-4
    x, a, b = torch.randn(T, n, generator=g), torch.randn(T, n, generator=g) * 5, torch.randn(T, n, generator=g) * 0.1
    wa, wb, w = torch.randn(n, generator=g), torch.randn(n, generator=g), torch.randn(n, generator=g)
    # two branches, each normed with its gain, half their sum, the scaled stream, the norm after it
    want = plain.norm(3.0 * x.double() + 0.5 * (plain.norm(a.double(), wa.double(), eps) + plain.norm(b.double(), wb.double(), eps)),
                      w.double(), eps)
    xs = x.to(DEV)
    copy = torch.empty((T, n), dtype=torch.bfloat16, device=DEV)
    ops.sum_norm(xs, [a.to(DEV), b.to(DEV)], [wa.to(DEV), wb.to(DEV)], w.to(DEV), eps, alpha=3.0, weight=0.5, copy=copy)
    _close(xs, want, 1e-5)
    _close(copy, want, 1e-2)
    # one branch as it is (a feed-forward's output)
    xs = x.to(DEV)
    ops.sum_norm(xs, [a.to(DEV)], [None], w.to(DEV), eps, alpha=1.0)
    _close(xs, plain.norm(x.double() + a.double(), w.double(), eps), 1e-5)
    # no norm after the sum, and a target that is only written (it may hold anything)
    xs = torch.full((T, n), float("nan"), device=DEV)
    ops.sum_norm(xs, [a.to(DEV), b.to(DEV)], [wa.to(DEV), None], None, eps, alpha=0.0, weight=2.0)
    _close(xs, 2.0 * (plain.norm(a.double(), wa.double(), eps) + b.double()), 1e-5)
