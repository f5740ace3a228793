"""Each mechanism of the Dokulix layers alone, kernel against the plain functions: the attention
kernel's blocks of positions, distance slopes, sink, value size and values read from the key rows
(with one key made to stand out far away, at page borders and just inside and outside every edge),
the latent preparation, the rotation of a part of every head, the per-head products, the gate, the
row vector, the gated activations, biased projections into the cache, norms stored around zero."""
import math

import pytest
import torch

from tests.plain import dokulix_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PAGE = 64


def _paged(rows: torch.Tensor, n_pages: int, perm: torch.Tensor, transposed: bool):
    """``rows [T, H, D]`` of one sequence into pool pages ``perm[0], perm[1], ...``."""
    T, H, D = rows.shape
    pool = torch.zeros((n_pages, H, D, PAGE) if transposed else (n_pages, H, PAGE, D), dtype=rows.dtype)
    for j in range(T):
        page = int(perm[j // PAGE])
        if transposed:
            pool[page, :, :, j % PAGE] = rows[j]
        else:
            pool[page, :, j % PAGE, :] = rows[j]
    return pool


def _attend(q, k, v, scale, visible, slopes, sink):
    """Plain attention of all positions of one sequence: q [T, H, D], k [T, G, D], v [T, G, Dv]."""
    T, H, _ = q.shape
    rep = H // k.shape[1]
    k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    if slopes is not None:
        dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).float()
        s = s - slopes[:, None, None] * dist[None]
    p = plain.softmax_visible(s, visible[None], sink)
    return torch.einsum("hij,jhd->ihd", p, v)


def _run_attention(q, k, v, scale, dtype, queries, window=None, chunk=None, slopes=None, sink=False, in_keys=False):
    """The kernel on the queries at ``queries`` (positions) over a cache that holds all T keys."""
    from rocml_amd import ops
    T, H, D = q.shape
    G = k.shape[1]
    dv = v.shape[2]
    n_pages = (T + PAGE - 1) // PAGE + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(T))
    kc = _paged(k, n_pages, perm, False).to(dtype).to(DEV)
    vc = None if in_keys else _paged(v, n_pages, perm, True).to(dtype).to(DEV)
    table = torch.full((1, 8), -1, dtype=torch.int32)
    table[0, :(T + PAGE - 1) // PAGE] = perm[:(T + PAGE - 1) // PAGE].to(torch.int32)
    qs = q[queries].reshape(len(queries), H * D).to(dtype).to(DEV).contiguous()
    out = torch.empty((len(queries), H * dv), dtype=dtype, device=DEV)
    seq = torch.zeros(len(queries), dtype=torch.int32, device=DEV)
    pos = torch.tensor(queries, dtype=torch.int32, device=DEV)
    ops.attention(qs, out, kc, vc, table.to(DEV), seq, pos, H, G, D, scale, window, v_head_dim=dv,
                  values_in_keys=in_keys, chunk=chunk, slopes=None if slopes is None else slopes.to(DEV), sink=sink)
    return out.float().cpu().view(len(queries), H, dv)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,G,D,DV,chunk", [(4, 2, 32, 16, 24), (3, 3, 16, 48, 65), (6, 1, 64, 64, 130), (2, 2, 20, 12, 1)])
def test_blocks_slopes_sink_and_value_size(dtype, tol, H, G, D, DV, chunk):
    gen = torch.Generator().manual_seed(D + chunk)
    T = 300
    q, k, v = torch.randn(T, H, D, generator=gen), torch.randn(T, G, D, generator=gen), torch.randn(T, G, DV, generator=gen)
    q, k, v = (t.to(torch.bfloat16).float() for t in (q, k, v))
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])
    scale = D ** -0.5
    queries = sorted(set([0, 1, chunk - 1, chunk, chunk + 1, 63, 64, 65, 2 * chunk - 1, 2 * chunk, 127, 128, 299]) & set(range(T)))
    for sl, sink in ((slopes, True), (None, True), (slopes, False)):
        ref = _attend(q, k, v, scale, plain.chunk_mask(T, chunk), sl, sink)[queries]
        got = _run_attention(q, k, v, scale, dtype, queries, chunk=chunk, slopes=sl, sink=sink)
        assert float((got - ref).abs().max()) < tol * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("edge", ["window", "chunk"])
def test_one_key_that_stands_out_at_every_edge(edge):
    """One key is made to carry nearly all the weight of a query that points at it; its value is large.
    Just inside the edge the output is that value, just outside it is not: an edge off by one, a page
    looked up wrongly or a far key lost shows as an error of order one."""
    T, H, D, size = 400, 2, 32, 70 if edge == "window" else 96
    gen = torch.Generator().manual_seed(5)
    base_k = 0.1 * torch.randn(T, 1, D, generator=gen)
    v = 0.1 * torch.randn(T, 1, D, generator=gen)
    for qpos in (size - 1, size, 191, 192, 193, 255, 256, 399):
        lo = max(0, qpos - size + 1) if edge == "window" else qpos - qpos % size
        for target in {lo - 1, lo, lo + 1, (lo // PAGE + 1) * PAGE - 1, (lo // PAGE + 1) * PAGE, qpos - 1, qpos}:
            if not 0 <= target <= qpos:
                continue
            k = base_k.clone()
            k[target] = 0.0
            k[target, 0, 3] = 6.0
            vv = v.clone()
            vv[target] = 50.0
            q = torch.zeros(T, H, D)
            q[qpos, :, 3] = 6.0 * D ** 0.5          # score 36 for the target, about zero for every other key
            visible = plain.window_mask(T, size) if edge == "window" else plain.chunk_mask(T, size)
            ref = _attend(q, k, vv, D ** -0.5, visible, None, edge == "chunk")[[qpos]]
            got = _run_attention(q, k, vv, D ** -0.5, torch.float32, [qpos], window=size if edge == "window" else None,
                                 chunk=size if edge == "chunk" else None, sink=edge == "chunk")
            assert float((got - ref).abs().max()) < 1e-3, f"query {qpos}, key {target}"
            assert (float(ref.abs().max()) > 40.0) == (target >= lo), "the oracle itself: inside means seen"


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
def test_values_read_from_the_key_rows(dtype, tol):
    """One shared key/value head whose values are the leading numbers of its key rows, under a window."""
    gen = torch.Generator().manual_seed(9)
    T, H, D, DV, window = 230, 5, 48, 40, 33
    q, k = torch.randn(T, H, D, generator=gen), torch.randn(T, 1, D, generator=gen)
    q, k = q.to(torch.bfloat16).float(), k.to(torch.bfloat16).float()
    queries = [0, 31, 32, 33, 34, 63, 64, 65, 96, 97, 229]
    ref = _attend(q, k, k[:, :, :DV], 0.2, plain.window_mask(T, window), None, False)[queries]
    got = _run_attention(q, k, k[:, :, :DV], 0.2, dtype, queries, window=window, in_keys=True)
    assert float((got - ref).abs().max()) < tol * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("q_rank,kv_rank,part,dims", [(48, 40, 8, 8), (32, 24, 16, 8), (12, 14, 6, 6), (300, 520, 64, 64)])
def test_latent_preparation(dtype, tol, q_rank, kv_rank, part, dims):
    from rocml_amd import ops
    gen = torch.Generator().manual_seed(q_rank)
    T, extra = 70, 5
    proj = torch.randn(T, q_rank + kv_rank + part + extra, generator=gen)
    qg, kg = 1 + 0.3 * torch.randn(q_rank, generator=gen), 1 + 0.3 * torch.randn(kv_rank, generator=gen)
    positions = torch.arange(100, 100 + T)
    eps, base = 1e-3, 777.0
    ref_q = plain.norm_plain(proj[:, :q_rank], qg, eps)
    ref_row = torch.cat([plain.norm_plain(proj[:, q_rank:q_rank + kv_rank], kg, eps),
                         plain.rotate_halves(proj[:, q_rank + kv_rank:q_rank + kv_rank + part], positions, base, dims)], dim=1)
    inv = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64, device=DEV)
    cos = torch.empty((T, dims // 2), dtype=torch.float32, device=DEV)
    sin = torch.empty_like(cos)
    pos = positions.to(torch.int32).to(DEV)
    ops.rope_table(pos, inv, cos, sin)
    cq = torch.empty((T, q_rank), dtype=dtype, device=DEV)
    cache = torch.zeros((4, PAGE, kv_rank + part), dtype=dtype, device=DEV)
    table = torch.tensor([[-1, 2, 0, 3]], dtype=torch.int32, device=DEV)     # positions 100 .. 169 lie in pages 1 and 2
    ops.latent_prepare(proj.to(DEV), q_rank, kv_rank, part, dims, qg.to(DEV), kg.to(DEV), eps, cos, sin, cq, cache, table,
                       torch.zeros(T, dtype=torch.int32, device=DEV), pos)
    assert float((cq.float().cpu() - ref_q).abs().max()) < tol * float(ref_q.abs().max())
    got = torch.cat([cache[2, 100 - 64:], cache[0, :170 - 128]]).float().cpu()
    assert float((got - ref_row).abs().max()) < tol * float(ref_row.abs().max())
    assert float(cache[3].abs().max()) == 0.0 and float(cache[1].abs().max()) == 0.0


@pytest.mark.parametrize("dims", [8, 4, 0])
def test_rotation_of_a_part_of_every_head(dims):
    from rocml_amd import ops
    gen = torch.Generator().manual_seed(3)
    T, H, d, part = 19, 3, 10, 8
    q = torch.randn(T, H, d + part, generator=gen)
    positions = torch.arange(5, 5 + T)
    ref = plain.rotate_halves(q[..., d:], positions, 50.0, dims) if dims else q[..., d:]
    cos = sin = None
    if dims:
        inv = torch.tensor([50.0 ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64, device=DEV)
        cos = torch.empty((T, dims // 2), dtype=torch.float32, device=DEV)
        sin = torch.empty_like(cos)
        ops.rope_table(positions.to(torch.int32).to(DEV), inv, cos, sin)
    out = torch.zeros((T, H * 20), dtype=torch.float32, device=DEV)
    ops.rope_heads(q.view(T, -1).to(DEV), H, d + part, d, part, dims, cos, sin, out, 20, 12)
    out = out.cpu().view(T, H, 20)
    assert float((out[..., 12:] - ref).abs().max()) < 1e-5
    assert float(out[..., :12].abs().max()) == 0.0


@pytest.mark.parametrize("tx,tw,to,tol", [(torch.float32, torch.float32, torch.float32, 1e-5),
                                          (torch.float32, torch.bfloat16, torch.bfloat16, 1e-2),
                                          (torch.bfloat16, torch.bfloat16, torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("T,H,K,N", [(1, 3, 10, 14), (70, 4, 16, 40), (130, 2, 65, 9)])
def test_per_head_products(tx, tw, to, tol, T, H, K, N):
    from rocml_amd import ops
    gen = torch.Generator().manual_seed(T + K)
    xs, os_ = K + 3, N + 2
    x = torch.randn(T, H * xs, generator=gen).to(tx)
    w = torch.randn(H, N, K, generator=gen).to(tw)
    out = torch.zeros((T, H * os_), dtype=to, device=DEV)
    ops.gemm_batched(x.to(DEV), xs, w.to(DEV), out, os_)
    ref = torch.einsum("thk,hnk->thn", x.float().view(T, H, xs)[..., :K], w.float())
    got = out.float().cpu().view(T, H, os_)
    assert float((got[..., :N] - ref).abs().max()) < tol * float(ref.abs().max())
    assert float(got[..., N:].abs().max()) == 0.0


def test_gate_row_vector_and_gated_activations():
    from rocml_amd import ops
    gen = torch.Generator().manual_seed(1)
    T, n = 37, 50
    y, g = torch.randn(T, n, generator=gen), torch.randn(T, n + 7, generator=gen)
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2)):
        yy = y.to(dtype).to(DEV)
        ops.sigmoid_gate(yy, g.to(DEV)[:, 7:])
        assert float((yy.float().cpu() - y.to(dtype).float() * torch.sigmoid(g[:, 7:])).abs().max()) < tol * 4
    x, b = torch.randn(T, n, generator=gen), torch.randn(n, generator=gen)
    xx = x.to(DEV)
    ops.add_row_vector(xx, b.to(DEV))
    assert torch.equal(xx.cpu(), x + b)
    gu = torch.randn(T, 2 * n, generator=gen)
    acts = {"silu": torch.nn.functional.silu, "relu": torch.relu,
            "gelu_tanh": lambda z: 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))}
    for name, fn in acts.items():
        for inter in (False, True):
            out = torch.empty((T, n), dtype=torch.float32, device=DEV)
            ops.swiglu(gu.to(DEV), out, interleaved=inter, activation=name)
            gate, up = (gu[:, 0::2], gu[:, 1::2]) if inter else (gu[:, :n], gu[:, n:])
            assert float((out.cpu() - fn(gate) * up).abs().max()) < 1e-5, name


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("m", [1, 5, 16, 40, 64, 200, 1100])
def test_relu_gated_product(dtype, tol, m):
    """Every kernel of the gate/up product has the rectifier as its epilogue."""
    from rocml_amd import ops
    gen = torch.Generator().manual_seed(m)
    k, inter = 128, 96
    x = torch.randn(m, k, generator=gen).to(dtype)
    gate, up = torch.randn(inter, k, generator=gen).to(dtype), torch.randn(inter, k, generator=gen).to(dtype)
    w = torch.stack([gate, up], dim=1).reshape(2 * inter, k).contiguous()
    out = torch.empty((m, inter), dtype=dtype, device=DEV)
    ws = torch.empty(1 << 22, dtype=torch.uint8, device=DEV)
    ops.gemm(x.to(DEV), w.to(DEV), out, workspace=ws, epilogue="relu_glu")
    ref = torch.relu(x.float() @ gate.float().T) * (x.float() @ up.float().T)
    assert float((out.float().cpu() - ref).abs().max()) < tol * float(ref.abs().max())


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("T", [3, 150])
@pytest.mark.parametrize("D,DV", [(32, 80), (128, 128)])
def test_biased_projection_rows_into_the_cache(dtype, tol, T, D, DV):
    """q and k rows get bias and per-head norm, v rows (of another size) their bias; k and v land in the pages."""
    from rocml_amd import ops
    gen = torch.Generator().manual_seed(T)
    H, G = 4, 2
    ld = (H + G) * D + G * DV
    qkv, bias = torch.randn(T, ld, generator=gen), torch.randn(ld, generator=gen)
    qg, kg = 1 + 0.3 * torch.randn(D, generator=gen), 1 + 0.3 * torch.randn(D, generator=gen)
    eps = 1e-4
    full = qkv + bias
    ref_q = plain.norm_plain(full[:, :H * D].view(T, H, D), qg, eps)
    ref_k = plain.norm_plain(full[:, H * D:(H + G) * D].view(T, G, D), kg, eps)
    ref_v = full[:, (H + G) * D:].view(T, G, DV)
    q_out = torch.empty((T, H * D), dtype=dtype, device=DEV)
    kc = torch.zeros((5, G, PAGE, D), dtype=dtype, device=DEV)
    vc = torch.zeros((5, G, DV, PAGE), dtype=dtype, device=DEV)
    table = torch.tensor([[4, 1, 3, 0]], dtype=torch.int32, device=DEV)
    pos = torch.arange(30, 30 + T, dtype=torch.int32, device=DEV)
    ops.qk_norm_rope_append(qkv.to(DEV), H, G, D, qg.to(DEV), kg.to(DEV), eps, None, None, 0, q_out, kc, vc, table,
                            torch.zeros(T, dtype=torch.int32, device=DEV), pos, bias=bias.to(DEV), v_head_dim=DV)
    assert float((q_out.float().cpu().view(T, H, D) - ref_q).abs().max()) < tol * float(ref_q.abs().max())
    pages = [4, 1, 3, 0]
    got_k = torch.stack([kc[pages[p // PAGE], :, p % PAGE, :] for p in range(30, 30 + T)]).float().cpu()
    got_v = torch.stack([vc[pages[p // PAGE], :, :, p % PAGE] for p in range(30, 30 + T)]).float().cpu()
    assert float((got_k - ref_k).abs().max()) < tol * float(ref_k.abs().max())
    assert float((got_v - ref_v).abs().max()) < tol * float(ref_v.abs().max())


def test_norm_whose_weight_is_stored_around_zero():
    from rocml_amd.config.spec import NormSpec
    from rocml_amd.parts import BuildContext, build_norm
    gen = torch.Generator().manual_seed(2)
    x, w = torch.randn(9, 40, generator=gen), 0.3 * torch.randn(40, generator=gen)
    ctx = BuildContext(dtype=torch.float32, device=torch.device(DEV))
    for offset, ref in ((True, plain.norm_one_plus(x, w, 1e-5)), (False, plain.norm_plain(x, w, 1e-5))):
        norm = build_norm(NormSpec(size=40, eps=1e-5, unit_offset=offset), ctx)
        norm.bind({"weight": w.to(DEV)})
        out = torch.empty((9, 40), dtype=torch.float32, device=DEV)
        norm.forward(x.to(DEV), out)
        assert float((out.cpu() - ref).abs().max()) < 1e-5


def _run_fast_attention(q, k, v, scale, first, window=None, chunk=None, slopes=None, sink=False, decode=False, n_splits=0):
    """The matrix-core kernels (bfloat16): the queries at positions ``first ..`` of one sequence as one
    prompt step, or, with ``decode``, each as the one new token of a sequence of its own."""
    from rocml_amd import ops
    T, H, D = q.shape
    G = k.shape[1]
    n_pages = (T + PAGE - 1) // PAGE + 2
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(T + first))
    kc = _paged(k, n_pages, perm, False).to(torch.bfloat16).to(DEV)
    vc = _paged(v, n_pages, perm, True).to(torch.bfloat16).to(DEV)
    n = T - first
    rows = n if decode else 1
    table = torch.full((rows, 8), -1, dtype=torch.int32)
    table[:, :(T + PAGE - 1) // PAGE] = perm[:(T + PAGE - 1) // PAGE].to(torch.int32)
    qs = q[first:].reshape(n, H * D).to(torch.bfloat16).to(DEV).contiguous()
    out = torch.empty((n, H * D), dtype=torch.bfloat16, device=DEV)
    seq = (torch.arange(n) if decode else torch.zeros(n)).to(torch.int32).to(DEV)
    pos = torch.arange(first, T, dtype=torch.int32, device=DEV)
    cu = (torch.arange(n + 1) if decode else torch.tensor([0, n])).to(torch.int32).to(DEV)
    ws = torch.empty(1 << 24, dtype=torch.uint8, device=DEV)
    ops.attention(qs, out, kc, vc, table.to(DEV), seq, pos, H, G, D, scale, window, algo=ops.ATTN_MFMA, workspace=ws,
                  cu_seqlens=cu, max_new=1 if decode else n, q_counts=[1] * n if decode else [n], max_len=T,
                  n_splits=n_splits, chunk=chunk, slopes=None if slopes is None else slopes.to(DEV), sink=sink)
    return out.float().cpu().view(n, H, D)


@pytest.mark.parametrize("H,G,D,chunk", [(8, 2, 64, 100), (6, 1, 96, 130), (4, 4, 128, 64), (2, 2, 32, 7)])
@pytest.mark.parametrize("decode", [False, True])
def test_matrix_core_kernels_take_blocks_slopes_and_sink(H, G, D, chunk, decode):
    gen = torch.Generator().manual_seed(H * D + chunk)
    T = 333
    q, k, v = (torch.randn(T, n, D, generator=gen).to(torch.bfloat16).float() for n in (H, G, G))
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])
    scale = D ** -0.5
    for first, sl, sink, splits in ((0, slopes, True, 0), (150, None, True, 3), (40, slopes, False, 1)):
        ref = _attend(q, k, v, scale, plain.chunk_mask(T, chunk), sl, sink)[first:]
        got = _run_fast_attention(q, k, v, scale, first, chunk=chunk, slopes=sl, sink=sink, decode=decode, n_splits=splits)
        err = (got - ref).abs().amax(dim=(1, 2))
        assert float(err.max()) < 2e-2 * max(1.0, float(ref.abs().max())), f"position {first + int(err.argmax())}"
    # and what they did before: a window, no extras
    ref = _attend(q, k, v, scale, plain.window_mask(T, 70), None, False)[20:]
    got = _run_fast_attention(q, k, v, scale, 20, window=70, decode=decode)
    assert float((got - ref).abs().max()) < 2e-2 * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("H,DK,DV,window", [(5, 48, 40, 33), (16, 96, 64, 100), (8, 192, 128, None), (16, 576, 512, 70), (3, 320, 256, 64)])
@pytest.mark.parametrize("decode", [False, True])
def test_matrix_core_kernel_for_latent_rows(H, DK, DV, window, decode):
    """Two sequences of unequal lengths whose rows of work (token, head) share one key/value head with the
    values in the key rows; a prompt step on top of cached positions, and a decode step."""
    from rocml_amd import ops
    gen = torch.Generator().manual_seed(H + DK)
    lens, firsts = (300, 131), ((0, 37) if not decode else (299, 130))
    n_pages = 12
    perm = torch.randperm(n_pages, generator=gen)
    cache = torch.zeros((n_pages, PAGE, DK), dtype=torch.bfloat16)
    table = torch.full((2, 8), -1, dtype=torch.int32)
    qs, refs, pos, seq, at = [], [], [], [], 0
    for b, (T, first) in enumerate(zip(lens, firsts)):
        q = torch.randn(T, H, DK, generator=gen).to(torch.bfloat16).float()
        k = torch.randn(T, 1, DK, generator=gen).to(torch.bfloat16).float()
        pages = perm[at:at + (T + PAGE - 1) // PAGE]
        at += len(pages)
        table[b, :len(pages)] = pages.to(torch.int32)
        for j in range(T):
            cache[int(pages[j // PAGE]), j % PAGE] = k[j, 0].to(torch.bfloat16)
        visible = plain.window_mask(T, window) if window else plain.window_mask(T, T)
        refs.append(_attend(q, k, k[:, :, :DV], DK ** -0.5, visible, None, False)[first:])
        qs.append(q[first:])
        pos += list(range(first, T))
        seq += [b] * (T - first)
    n = len(pos)
    qd = torch.cat(qs).reshape(n, H * DK).to(torch.bfloat16).to(DEV).contiguous()
    out = torch.empty((n, H * DV), dtype=torch.bfloat16, device=DEV)
    counts = [T - f for T, f in zip(lens, firsts)]
    cu = torch.tensor([0, counts[0], n], dtype=torch.int32, device=DEV)
    ws = torch.empty(1 << 26, dtype=torch.uint8, device=DEV)
    ops.attention(qd, out, cache.to(DEV).unsqueeze(1), None, table.to(DEV), torch.tensor(seq, dtype=torch.int32, device=DEV),
                  torch.tensor(pos, dtype=torch.int32, device=DEV), H, 1, DK, DK ** -0.5, window, algo=ops.ATTN_MFMA,
                  workspace=ws, cu_seqlens=cu, max_new=max(counts), q_counts=counts, max_len=max(lens),
                  v_head_dim=DV, values_in_keys=True)
    got, ref = out.float().cpu().view(n, H, DV), torch.cat(refs)
    err = (got - ref).abs().amax(dim=(1, 2))
    assert float(err.max()) < 2e-2 * max(1.0, float(ref.abs().max())), f"row {int(err.argmax())}, position {pos[int(err.argmax())]}"


@pytest.mark.parametrize("tx", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,K,N,xs,os_", [(1, 3, 16, 24, 24, 32), (8, 16, 128, 512, 192, 576), (70, 4, 40, 20, 48, 20),
                                            (300, 2, 512, 128, 512, 128), (17, 6, 64, 32, 64, 32)])
def test_per_head_products_on_the_matrix_cores(tx, T, H, K, N, xs, os_):
    """bfloat16 weights, strides that 16-byte loads reach: the matrix-core kernel; with the gate as its epilogue
    where the output has no gaps."""
    from rocml_amd import ops
    gen = torch.Generator().manual_seed(T + K + N)
    x = torch.randn(T, H * xs, generator=gen).to(tx)
    w = (torch.randn(H, N, K, generator=gen) * K ** -0.5).to(torch.bfloat16)
    ref = torch.einsum("thk,hnk->thn", x.float().view(T, H, xs)[..., :K], w.float())
    gate = torch.randn(T, 7 + H * N, generator=gen)
    for use_gate in (False, True):
        if use_gate and os_ != N:
            continue
        out = torch.zeros((T, H * os_), dtype=torch.bfloat16, device=DEV)
        ops.gemm_batched(x.to(DEV), xs, w.to(DEV), out, os_, gate=gate.to(DEV)[:, 7:] if use_gate else None)
        want = ref * torch.sigmoid(gate[:, 7:].view(T, H, N)) if use_gate else ref
        got = out.float().cpu().view(T, H, os_)
        assert float((got[..., :N] - want).abs().max()) < 1.5e-2 * float(want.abs().max())
        assert os_ == N or float(got[..., N:].abs().max()) == 0.0
