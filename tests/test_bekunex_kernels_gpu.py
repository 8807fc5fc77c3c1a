"""The kernels that the Bekunex decoder added, each alone against the plain formulas
(``plain_bekunex.py``, float64): layer norm with the residual add, one product per head, the
latent's norm / rotation / cache write and the attention over cached latents (window, sink,
pages in any order), the sigmoid gate, the choice of experts and the routed units (tiles of 16
and of 64 rows), the selective scan with its state carried over steps, and the convolution's
bias."""
import pytest
import torch

import plain_bekunex as plain

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda", 0)
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def rel(got, want):
    want = want.double().cpu()
    return float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-9))


def rnd(*shape, seed=0, std=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed + 1000 * len(shape) + sum(shape))
    return (torch.randn(shape, generator=g) * std).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [40, 192, 1000])
def test_layer_norm_with_the_residual_add(dtype, width):
    from rust_llm_inference_server_amd import ops
    T = 7
    resid, delta = rnd(T, width, seed=1) * 3 + 1.5, rnd(T, width, seed=2).to(dtype)
    w, b = (1 + rnd(width, seed=3, std=0.3)).to(dtype), rnd(width, seed=4, std=0.2).to(dtype)
    want_sum = resid.double() + delta.double()
    want = plain.layer_norm(want_sum, w.double(), b.double(), 1e-5)
    r = resid.to(DEV).clone()
    got = ops.add_layernorm(r, delta.to(DEV), w.to(DEV), b.to(DEV), 1e-5, dtype)
    assert rel(got, want) < TOL[dtype]
    assert rel(r, want_sum) < 1e-6                       # the sum is stored back, in float32
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    r2 = resid.to(DEV).clone()
    got = ops.add_layernorm(r2, delta.to(DEV), w.to(DEV), b.to(DEV), 1e-5, dtype, rows=rows)
    assert rel(got, want[[5, 0, 5]]) < TOL[dtype]
    assert torch.equal(r2.cpu(), resid)                  # a selection leaves the residual
    got = ops.add_layernorm(r2, None, w.to(DEV), b.to(DEV), 1e-5, torch.float32)
    assert rel(got, plain.layer_norm(resid.double(), w.double(), b.double(), 1e-5)) < 2e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, N, K, pad", [(3, 40, 16, 8), (2, 28, 12, 6), (5, 100, 72, 0),
                                          (1, 16, 130, 3)])
@pytest.mark.parametrize("T", [1, 37, 150])
def test_one_product_per_head(dtype, H, N, K, pad, T):
    """Heads that lie ``K + pad`` apart in the rows of x, results written ``N + pad`` apart into
    a given tensor whose other columns stay; sizes on and off the 16-byte loads."""
    from rust_llm_inference_server_amd import ops
    x = rnd(T, H * (K + pad), seed=5).to(dtype)
    w = rnd(H, N, K, seed=6, std=K ** -0.5).to(dtype)
    out = torch.full((T, H * (N + pad)), 7.0, dtype=dtype, device=DEV)
    ops.head_linear(x.to(DEV), w.to(DEV), K + pad, out=out, out_head=N + pad)
    xs = x.double().reshape(T, H, K + pad)[..., :K]
    want = torch.einsum("thk,hnk->thn", xs, w.double())
    got = out.reshape(T, H, N + pad)
    assert rel(got[..., :N], want) < TOL[dtype]
    assert bool((got[..., N:] == 7.0).all())
    fresh = ops.head_linear(x.to(DEV), w.to(DEV), K + pad)
    assert torch.equal(fresh.reshape(T, H, N), got[..., :N].contiguous())


def _cached_attention_case(dtype, H, d, r, R, n, page, seed):
    """Queries of one sequence of n positions, their down projections, and random maps."""
    q = rnd(n, H * (d + r), seed=seed).to(dtype)
    down = rnd(n, R + r, seed=seed + 1) * 2
    norm = 1 + rnd(R, seed=seed + 2, std=0.3)
    uk = rnd(H * d, R, seed=seed + 3, std=R ** -0.5).to(dtype)
    return q, down, norm, uk


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, d, r, R, window, sink", [
    (3, 16, 8, 40, None, False), (2, 12, 6, 28, None, False), (4, 8, 0, 36, 16, True),
    (1, 24, 0, 70, 1, True), (2, 16, 0, 16, 33, False), (2, 32, 16, 128, 17, True),
    (20, 16, 16, 64, None, False), (16, 8, 0, 200, 40, True), (5, 16, 32, 288, None, True),
    (2, 8, 8, 520, 50, True)])
def test_attention_over_cached_latents(dtype, H, d, r, R, window, sink, monkeypatch):
    """Cache write in two portions (pages in a shuffled order), then every query against the
    plain softmax over keys made from the latents: rotation, norm, window edges, the sink."""
    from rust_llm_inference_server_amd import ops
    n, page, base, scale, eps = 75, 16, 1000.0, 0.3, 1e-5
    D = R + r
    q, down, norm, uk = _cached_attention_case(dtype, H, d, r, R, n, page, seed=H + d)
    sink_w = rnd(H, seed=9) * 2 if sink else None
    pos = torch.arange(n)
    # the plain side: keys from the normed latent, the rotated part shared by the heads
    c = plain.rms_norm(down[:, :R].double(), norm.double(), eps)
    c_stored = c.to(dtype).double()                      # what the cache holds
    k = (c_stored @ uk.double().T).reshape(n, H, d)
    qd = q.double().reshape(n, H, d + r)
    if r:
        kr = plain.rotate(down[:, R:].double(), pos, r, base).to(dtype).double()
        qr = plain.rotate(qd[..., d:], pos, r, base)
        k = torch.cat([k, kr.reshape(n, 1, r).expand(n, H, r)], -1)
        qd = torch.cat([qd[..., :d], qr], -1)
    want = plain.softmax_attention(qd, k, c_stored.reshape(n, 1, R).expand(n, H, R), scale,
                                   window, None if sink_w is None else sink_w.double())
    # the engine's side
    num_pages = 9
    order = torch.randperm(num_pages, generator=torch.Generator().manual_seed(3))[:-(-n // page)]
    table = torch.zeros(1, 8, dtype=torch.int32)
    table[0, :len(order)] = order.to(torch.int32)
    slots = (table[0, pos // page].long() * page + pos % page).to(torch.int32)
    pages = torch.zeros(num_pages, page, D, dtype=dtype, device=DEV)
    matrix = ops.latent_mfma_ok(dtype, R, D, page)
    assert matrix == (dtype == torch.bfloat16 and D % 8 == 0)
    pages_t = torch.zeros(num_pages, R, page, dtype=dtype, device=DEV) if matrix else None
    cos = sin = None
    if r:
        ang = pos.double().reshape(-1, 1) * base ** (-torch.arange(0, r, 2).double() / r)
        cos, sin = (f(ang).float().to(DEV).contiguous() for f in (torch.cos, torch.sin))
    w_uk_t = uk.reshape(H, d, R).transpose(1, 2).contiguous().to(DEV)
    qg = q.to(DEV)
    q_lat = torch.zeros(n, H * D, dtype=dtype, device=DEV)
    ops.head_linear(qg, w_uk_t, d + r, out=q_lat, out_head=D)
    posd = pos.to(torch.int32).to(DEV)
    for lo, hi in ((0, 41), (41, n)):
        ops.latent_write(down[lo:hi].to(DEV), norm.to(DEV), eps, R, r, r, cos, sin, posd[lo:hi],
                         slots[lo:hi].to(DEV), pages, qg[lo:hi] if r else None, d + r,
                         q_lat[lo:hi] if r else None, H, pages_t)
    args = (q_lat, pages, table.to(DEV), torch.zeros(n, dtype=torch.int32, device=DEV), posd, H, R,
            scale, window, None if sink_w is None else sink_w.to(DEV))
    got = ops.latent_attention(*args)                    # the vector-unit kernel
    assert rel(got.reshape(n, H, R), want) < (3e-5 if dtype == torch.float32 else 3e-2)
    if matrix:
        assert torch.equal(pages_t.transpose(1, 2), pages[:, :, :R])
        cu = torch.tensor([0, n], dtype=torch.int32, device=DEV)
        from rust_llm_inference_server_amd.ops import latent
        # a workgroup's waves share a block's keys; every wave loads for itself; a workgroup
        # stages a chunk once for four blocks
        for blocks, staged in ((1024, False), (0, False), (0, True)):
            monkeypatch.setattr(latent, "LATENT_SPLIT_MAX_BLOCKS", blocks)
            monkeypatch.setattr(latent, "LATENT_STAGED", staged)
            got = ops.latent_attention(*args, pages_t=pages_t, cu=cu, num_seqs=1)
            assert rel(got.reshape(n, H, R), want) < 3e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sigmoid_gate_in_place_on_rows_of_any_stride(dtype):
    from rust_llm_inference_server_amd import ops
    o, g = rnd(9, 40, seed=1).to(dtype), rnd(9, 100, seed=2).to(dtype)
    og = o.to(DEV)
    ops.sigmoid_gate_(og, g.to(DEV)[:, 30:70])
    assert rel(og, o.double() * torch.sigmoid(g.double()[:, 30:70])) < TOL[dtype]


@pytest.mark.parametrize("E, G, keep, top", [(8, 2, 1, 4), (6, 3, 2, 3), (4, 1, 1, 1),
                                             (3, 3, 3, 3), (64, 8, 3, 6), (130, 5, 2, 9)])
def test_the_choice_of_experts(E, G, keep, top):
    """Groups by the sum of their two best choice scores, the correction in the choice only,
    weights from the scores without it; negative choice scores in the groups left out."""
    from rust_llm_inference_server_amd import ops
    T, W = 50, 24
    h = rnd(T, W, seed=E)
    weights = {"m.router": rnd(E, W, seed=E + 1, std=0.6), "m.correction": rnd(E, seed=E + 2) - 0.8}
    router = {"experts": E, "top": top, "groups": {"count": G, "keep": keep}, "scale": 1.7}
    want_idx, want_w = plain.route(h.double(), weights, "m", router)
    logits = (h.double() @ weights["m.router"].double().T).float().to(DEV)
    idx, w = ops.route(logits, weights["m.correction"].to(DEV), G, keep, top, 1.7)
    assert torch.equal(idx.cpu().long().sort(1).values, want_idx.sort(1).values)
    order = idx.cpu().long().argsort(1)
    assert rel(w.cpu().gather(1, order), want_w.gather(1, want_idx.argsort(1))) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T, W, E", [(1, 40, 3), (9, 192, 8), (70, 1000, 33)])
def test_router_logits_from_the_residual(dtype, T, W, E):
    """Layer norm and the router's product in one kernel, float32 on weights of either dtype."""
    from rust_llm_inference_server_amd import ops
    resid = rnd(T, W, seed=1) * 3 + 0.5
    w, b = (1 + rnd(W, seed=2, std=0.3)).to(dtype), rnd(W, seed=3, std=0.2).to(dtype)
    router = rnd(E, W, seed=4, std=W ** -0.5).to(dtype)
    want = plain.layer_norm(resid.double(), w.double(), b.double(), 1e-5) @ router.double().T
    got = ops.router_logits(resid.to(DEV), w.to(DEV), b.to(DEV), 1e-5, router.to(DEV))
    assert got.dtype == torch.float32 and rel(got, want) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T, E, top, W, F", [(1, 4, 2, 48, 24), (9, 8, 3, 40, 20),
                                             (200, 6, 2, 64, 32), (77, 3, 1, 36, 12),
                                             (700, 4, 2, 72, 40), (1000, 3, 3, 200, 136)])
def test_routed_units(dtype, T, E, top, W, F):
    """Tiles of 16 rows (few pairs), of 64 (many) and, in bfloat16, of 128 through LDS (very
    many), widths on and off the 16-byte loads and the tiles' sizes, with and without an addend;
    experts that no token chose."""
    from rust_llm_inference_server_amd import ops
    x = rnd(T, W, seed=T).to(dtype)
    wgu = rnd(E, 2 * F, W, seed=T + 1, std=W ** -0.5).to(dtype)
    wd = rnd(E, W, F, seed=T + 2, std=F ** -0.5).to(dtype)
    g = torch.Generator().manual_seed(T)
    chosen = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    if top == 1:
        chosen[chosen == 1] = 0                          # an expert that no token chose
    wts = torch.rand(T, top, generator=g) + 0.2
    add = rnd(T, W, seed=T + 3).to(dtype)
    want = torch.zeros(T, W, dtype=torch.float64)
    for t in range(T):
        for e, wt in zip(chosen[t].tolist(), wts[t].tolist()):
            gu = wgu[e].double() @ x[t].double()
            hidden = (plain.silu(gu[:F]) * gu[F:]).to(dtype).double()
            want[t] += wt * (wd[e].double() @ hidden)
    args = (x.to(DEV), wgu.to(DEV), wd.to(DEV), chosen.to(DEV), wts.to(DEV))
    got = ops.routed_units(*args)
    assert got.dtype == torch.float32 and rel(got, want) < TOL[dtype]
    got = ops.routed_units(*args, add.to(DEV))
    assert rel(got, want + add.double()) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C, N", [(24, 5), (64, 16), (40, 20), (33, 64), (16, 70), (8, 300)])
@pytest.mark.parametrize("chunked", [False, True])
def test_selective_scan_carries_its_state(dtype, C, N, chunked, monkeypatch):
    """Two sequences in one step, then their continuations in a second step with the slots
    swapped in the batch's order: the same as each sequence in one pass.  ``chunked``: the form
    for long prompts, here with chunks of 4 tokens, so that sequences of 2 to 13 tokens are
    one chunk, several whole ones, and some with a short last one."""
    from rust_llm_inference_server_amd import ops
    from rust_llm_inference_server_amd.ops import recurrent
    if chunked:
        monkeypatch.setattr(recurrent, "CHUNKED_SCAN_MIN_TOKENS", 0)
        monkeypatch.setattr(recurrent, "CHUNKED_SCAN_MIN_MEAN_TOKENS", 0)
        monkeypatch.setattr(recurrent, "CHUNKED_SCAN_LEN", 4)
    lens = [(9, 6), (2, 13)]
    total = [a + b for a, b in lens]
    data = []
    for s, n in enumerate(total):
        data.append(dict(x=rnd(n, C, seed=s).to(dtype), dt=rnd(n, C, seed=s + 10),
                         b=rnd(n, N, seed=s + 20), c=rnd(n, N, seed=s + 30),
                         z=rnd(n, C, seed=s + 40)))
    bias, a_log, skip = rnd(C, seed=50) - 1, rnd(C, N, seed=51) - 1, rnd(C, seed=52)
    want = []
    for d in data:
        S = torch.zeros(C, N, dtype=torch.float64)
        dt = torch.nn.functional.softplus(d["dt"].double() + bias.double())
        A = -torch.exp(a_log.double())
        rows = []
        for t in range(d["x"].shape[0]):
            xv = d["x"][t].double()
            S = torch.exp(dt[t].reshape(C, 1) * A) * S + (dt[t] * xv).reshape(C, 1) * d["b"][t].double()
            rows.append((S @ d["c"][t].double() + skip.double() * xv) * plain.silu(d["z"][t].double()))
        want.append(torch.stack(rows))
    state = torch.zeros(3, C * N + 4, dtype=torch.float32, device=DEV)[:, :C * N]
    got = [[], []]
    for step, order in ((0, (0, 1)), (1, (1, 0))):
        parts = {k: [] for k in ("x", "dt", "b", "c", "z")}
        cu = [0]
        for s in order:
            lo = 0 if step == 0 else lens[s][0]
            hi = lens[s][0] if step == 0 else total[s]
            for k in parts:
                parts[k].append(data[s][k][lo:hi])
            cu.append(cu[-1] + hi - lo)
        cat = {k: torch.cat(v).to(DEV) for k, v in parts.items()}
        bc = torch.cat([cat["b"], cat["c"]], dim=1).contiguous()
        out = ops.selective_scan(cat["x"], cat["dt"], bias.to(DEV), bc[:, :N], bc[:, N:],
                                 cat["z"], a_log.to(DEV), skip.to(DEV), state,
                                 torch.tensor(cu, dtype=torch.int32, device=DEV),
                                 torch.tensor([2 if s == 0 else 0 for s in order],
                                              dtype=torch.int32, device=DEV), 2)
        for i, s in enumerate(order):
            got[s].append(out[cu[i]:cu[i + 1]])
    for s in range(2):
        assert rel(torch.cat(got[s]), want[s]) < TOL[dtype]
    assert float(state[1].abs().max()) == 0.0            # a slot that no sequence had


def test_the_convolutions_bias_and_output_dtype():
    from rust_llm_inference_server_amd import ops
    T, C, K = 11, 40, 3
    x, taps, bias = rnd(T, C + 8, seed=1), rnd(C, K, seed=2), rnd(C, seed=3)
    state = torch.zeros(1, C * (K - 1), dtype=torch.float32, device=DEV)
    meta = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    padded = torch.cat([torch.zeros(K - 1, C), x[:, :C]]).double()
    acc = bias.double() + sum(padded[j:j + T] * taps[:, j].double() for j in range(K))
    for dtype in (torch.float32, torch.bfloat16):
        got = ops.causal_conv(x.to(DEV), taps.to(DEV), state, meta([0] * T), meta([0, T]),
                              meta([0]), 1, bias=bias.to(DEV), out_dtype=dtype)
        assert got.dtype == dtype and rel(got, plain.silu(acc)) < TOL[dtype]


@pytest.mark.parametrize("H, d, r, R, window", [(16, 16, 16, 128, None), (32, 8, 0, 288, 300),
                                                (3, 32, 0, 64, 77)])
def test_large_steps_of_both_attention_kernels_agree(H, d, r, R, window, monkeypatch):
    """Two sequences of 1,100 and 500 tokens in one step, behind 40 cached positions of the first:
    the matrix-core kernel in the forms it chooses by itself for a step of this size (staged, or
    a wave per block) against the vector-unit kernel, row by row."""
    from rust_llm_inference_server_amd import ops
    from rust_llm_inference_server_amd.ops import latent
    dtype, page, D = torch.bfloat16, 16, R + r
    lens, starts = [1100, 500], [40, 0]
    total = [a + b for a, b in zip(lens, starts)]
    T = sum(lens)
    pages_needed = [-(-n // page) for n in total]
    num_pages = sum(pages_needed) + 3
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(5))
    table = torch.zeros(2, 128, dtype=torch.int32)
    table[0, :pages_needed[0]] = perm[:pages_needed[0]].to(torch.int32)
    table[1, :pages_needed[1]] = perm[pages_needed[0]:sum(pages_needed)].to(torch.int32)
    pages = (rnd(num_pages, page, D, seed=11) * 0.7).to(dtype).to(DEV)
    pages_t = pages[:, :, :R].transpose(1, 2).contiguous()
    q = (rnd(T, H * D, seed=12) * 0.5).to(dtype).to(DEV)
    seq = torch.cat([torch.zeros(lens[0]), torch.ones(lens[1])]).to(torch.int32).to(DEV)
    pos = torch.cat([torch.arange(starts[0], total[0]),
                     torch.arange(starts[1], total[1])]).to(torch.int32).to(DEV)
    cu = torch.tensor([0, lens[0], T], dtype=torch.int32, device=DEV)
    sink = (rnd(H, seed=13)).to(DEV)
    args = (q, pages, table.to(DEV), seq, pos, H, R, 0.2, window, sink)
    want = ops.latent_attention(*args)
    for staged in (True, False):
        monkeypatch.setattr(latent, "LATENT_STAGED", staged)
        got = ops.latent_attention(*args, pages_t=pages_t, cu=cu, num_seqs=2)
        assert rel(got, want) < 2e-2
