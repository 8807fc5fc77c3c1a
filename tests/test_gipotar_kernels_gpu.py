"""Each new kernel alone against the plain formulas of ``plain_gipotar.py`` (float64), at sizes
the models of the other tests do not have: more than 64 and more than 128 key channels, value
sizes that are no multiple of a workgroup's columns, taps from 2 to 7, steps shorter than the
input tail, several sequences per step in state slots that are not in order, the state carried
over steps."""
import pytest
import torch

import plain_gipotar as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _ops():
    from rust_llm_inference_server_amd import ops
    return ops


def _meta(lengths, slots):
    cu = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32, device=DEV)
    seq = torch.repeat_interleave(torch.arange(len(lengths)), torch.tensor(lengths)).to(
        torch.int32).to(DEV)
    return cu, torch.tensor(slots, dtype=torch.int32, device=DEV), seq


def _state(num_slots, used, extra=24):
    """A state buffer whose rows are longer than the mixer's area, filled with garbage that the
    test clears for the slots it uses (as the runner does for a request at position 0)."""
    buf = torch.full((num_slots, used + extra), 7.5, dtype=torch.float32, device=DEV)
    return buf, buf[:, 8:8 + used]


# tokens per sequence, step by step (runs longer than a tile of the tiled scans among them, and
# runs that end one token short of a tile, at its end, and inside a group of tokens behind it)
STEPS = [[5, 1, 9], [1, 1, 2], [3, 1, 1], [17, 2, 1], [2, 70, 33], [31, 32, 34], [15, 16, 7]]
SLOTS = [3, 0, 2]


def _cut(x, lengths_by_step, step, seq):
    """Rows of sequence ``seq`` in step ``step`` within that sequence's own row order."""
    start = sum(l[seq] for l in lengths_by_step[:step])
    return slice(start, start + lengths_by_step[step][seq])


@pytest.mark.parametrize("tiled", [False, "wide", "narrow", None])
@pytest.mark.parametrize("heads, d", [(3, 16), (2, 96), (1, 160), (2, 50)])
def test_decayed_state_scan(heads, d, tiled):
    """``tiled``: the kernel that asks for a token's vectors one token ahead, the one that stages
    tiles of tokens through LDS with four or with two value channels a wave, or whichever the
    step's shape chooses."""
    ops = _ops()
    g = torch.Generator().manual_seed(heads * 100 + d)
    totals = [sum(s[i] for s in STEPS) for i in range(3)]
    data = [{n: torch.randn(T, heads * d, generator=g) * 0.5 for n in "rkvz"} for T in totals]
    w0 = torch.rand(heads * d, generator=g) * -4.0 - 0.5
    bonus = torch.randn(heads, d, generator=g) * 0.5
    buf, state = _state(4, heads * d * d)
    state[SLOTS] = 0.0
    want, S = [], []
    for x in data:
        Sx = torch.zeros(heads, d, d, dtype=torch.float64)
        decay = torch.exp(-torch.exp(x["z"].double() + w0.double()))
        want.append(plain.decayed_state(*(x[n].double().reshape(-1, heads, d) for n in "rkv"),
                                        decay.reshape(-1, heads, d), bonus.double(), Sx))
        S.append(Sx)
    for step, lengths in enumerate(STEPS):
        cu, slots, _ = _meta(lengths, SLOTS)
        rows = {n: torch.cat([data[i][n][_cut(None, STEPS, step, i)] for i in range(3)]).to(DEV)
                for n in "rkvz"}
        out = ops.decay_scan(rows["r"], rows["k"], rows["v"], rows["z"], w0.to(DEV),
                             bonus.to(DEV), state, cu, slots, 3, heads, d, tiled=tiled).cpu()
        at = 0
        for i, n in enumerate(lengths):
            ref = want[i][_cut(None, STEPS, step, i)].reshape(n, heads * d)
            assert torch.allclose(out[at:at + n].double(), ref, rtol=2e-4, atol=2e-4)
            at += n
    for i, slot in enumerate(SLOTS):                   # [head][value][key] in the slot
        got = state[slot].cpu().reshape(heads, d, d).transpose(1, 2).double()
        assert torch.allclose(got, S[i], rtol=2e-4, atol=2e-4)
    assert float(buf[1].min()) == 7.5 and float(buf[:, :8].min()) == 7.5     # nothing else moved


@pytest.mark.parametrize("tiled", [False, "wide", "narrow", None])
@pytest.mark.parametrize("heads, groups, dk, dv", [(4, 2, 16, 24), (2, 1, 96, 6), (1, 1, 200, 33),
                                                   (6, 3, 64, 64)])
def test_gated_delta_scan(heads, groups, dk, dv, tiled):
    ops = _ops()
    g = torch.Generator().manual_seed(dk * 10 + dv)
    totals = [sum(s[i] for s in STEPS) for i in range(3)]
    C = 2 * groups * dk + heads * dv
    a_log = torch.rand(heads, generator=g) * 3.0 - 3.0
    dt_bias = torch.rand(heads, generator=g) * 3.0 - 2.5
    data = []
    for T in totals:
        q = plain.unit(torch.randn(T, groups, dk, generator=g).double()) * dk ** -0.5
        k = plain.unit(torch.randn(T, groups, dk, generator=g).double())
        v = torch.randn(T, heads, dv, generator=g).double()
        ba = torch.randn(T, 2 * heads, generator=g).double() * 2.0
        data.append({"qkv": torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1),
                     "ba": ba, "q": q, "k": k, "v": v})
    buf, state = _state(4, heads * dv * dk)
    state[SLOTS] = 0.0
    want, S = [], []
    for x in data:
        Sx = torch.zeros(heads, dk, dv, dtype=torch.float64)
        beta = torch.sigmoid(x["ba"][:, :heads])
        decay = torch.exp(-torch.exp(a_log.double())
                          * plain.softplus(x["ba"][:, heads:] + dt_bias.double()))
        want.append(plain.delta_state(x["q"], x["k"], x["v"], beta, decay, Sx))
        S.append(Sx)
    for step, lengths in enumerate(STEPS):
        cu, slots, _ = _meta(lengths, SLOTS)
        qkv = torch.cat([data[i]["qkv"][_cut(None, STEPS, step, i)] for i in range(3)]).float().to(DEV)
        ba = torch.cat([data[i]["ba"][_cut(None, STEPS, step, i)] for i in range(3)]).float().to(DEV)
        out = ops.delta_scan(qkv[:, :groups * dk], qkv[:, groups * dk:2 * groups * dk],
                             qkv[:, 2 * groups * dk:], ba[:, :heads], ba[:, heads:],
                             a_log.to(DEV), dt_bias.to(DEV), state, cu, slots, 3, heads, groups,
                             dk, dv, tiled=tiled).cpu()
        at = 0
        for i, n in enumerate(lengths):
            ref = want[i][_cut(None, STEPS, step, i)].reshape(n, heads * dv)
            assert torch.allclose(out[at:at + n].double(), ref, rtol=2e-4, atol=2e-5)
            at += n
    for i, slot in enumerate(SLOTS):
        got = state[slot].cpu().reshape(heads, dv, dk).transpose(1, 2).double()
        assert torch.allclose(got, S[i], rtol=2e-4, atol=2e-5)
    assert C > 0 and float(buf[1].min()) == 7.5


@pytest.mark.parametrize("taps, unit_heads, dk, rest, dv", [(2, 2, 16, 3, 8), (4, 4, 48, 2, 40),
                                                            (7, 1, 300, 1, 5), (1, 2, 8, 1, 8)])
def test_short_convolution_with_tails_and_unit_vectors(taps, unit_heads, dk, rest, dv):
    """The first half of the unit heads is also scaled (queries), the second is not (keys)."""
    ops = _ops()
    g = torch.Generator().manual_seed(taps)
    unit_heads *= 2
    U, C = unit_heads * dk, unit_heads * dk + rest * dv
    totals = [sum(s[i] for s in STEPS) for i in range(3)]
    w = torch.randn(C, taps, generator=g) * 0.6
    xs = [torch.randn(T, C + 5, generator=g) for T in totals]          # wider rows than C
    want = []
    for x in xs:
        y = plain.silu(plain.short_conv(x[:, :C].double(), w.double()))
        u = plain.unit(y[:, :U].reshape(-1, unit_heads, dk)).reshape(-1, U)
        u[:, :U // 2] *= 0.3
        want.append(torch.cat([u, y[:, U:]], 1))
    buf, state = _state(4, C * (taps - 1))
    state[SLOTS] = 0.0
    for step, lengths in enumerate(STEPS):
        cu, slots, seq = _meta(lengths, SLOTS)
        x = torch.cat([xs[i][_cut(None, STEPS, step, i)] for i in range(3)]).to(DEV)
        out = ops.causal_conv(x, w.to(DEV), state, seq, cu, slots, 3, unit_channels=U,
                              unit_group=dk, scaled_channels=U // 2, scale=0.3, unit_eps=1e-6,
                              rest_group=dv).cpu()
        ops.tail_update(state, x, C, taps - 1, cu, slots, 3)
        at = 0
        for i, n in enumerate(lengths):
            ref = want[i][_cut(None, STEPS, step, i)]
            assert torch.allclose(out[at:at + n].double(), ref, rtol=1e-4, atol=1e-5)
            at += n
    assert float(buf[1].min()) == 7.5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_shift_blends(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(4)
    W, mixes = 72, 5
    totals = [sum(s[i] for s in STEPS) for i in range(3)]
    mu = torch.rand(mixes, W, generator=g)
    xs = [torch.randn(T, W, generator=g).to(dtype) for T in totals]
    buf, state = _state(4, W)
    state[SLOTS] = 0.0
    for step, lengths in enumerate(STEPS):
        cu, slots, seq = _meta(lengths, SLOTS)
        x = torch.cat([xs[i][_cut(None, STEPS, step, i)] for i in range(3)]).to(DEV)
        out = ops.shift_mix(x, mu.to(DEV), state, seq, cu, slots, 3).cpu()
        ops.tail_update(state, x, W, 1, cu, slots, 3)
        at = 0
        for i, n in enumerate(lengths):
            full = xs[i].double()
            prev = torch.cat([torch.zeros(1, W, dtype=torch.float64), full[:-1]])
            rows = _cut(None, STEPS, step, i)
            for m in range(mixes):
                ref = (full + (prev - full) * mu[m].double())[rows]
                tol = 1e-5 if dtype == torch.float32 else 2e-2
                assert torch.allclose(out[m, at:at + n].double(), ref, rtol=tol, atol=tol)
            at += n


@pytest.mark.parametrize("heads, dv, shared", [(3, 24, False), (2, 100, True), (1, 8, True)])
def test_head_norm_weight_and_gate(heads, dv, shared):
    ops = _ops()
    g = torch.Generator().manual_seed(dv)
    T = 11
    o = torch.randn(T, heads * dv, generator=g)
    gate = torch.randn(T, heads * dv + 8, generator=g)
    w = 1.0 + torch.randn(dv if shared else heads * dv, generator=g) * 0.3
    got = ops.head_norm_gate(o.to(DEV), w.to(DEV), gate.to(DEV)[:, 8:], heads, dv, 1e-5,
                             torch.float32).cpu().double()
    x = plain.rms(o.double().reshape(T, heads, dv), 1e-5)
    wd = w.double().reshape(1, 1, dv) if shared else w.double().reshape(1, heads, dv)
    ref = (x * wd * plain.silu(gate[:, 8:].double().reshape(T, heads, dv))).reshape(T, heads * dv)
    assert torch.allclose(got, ref, rtol=1e-5, atol=1e-6)


def test_clamped_gated_unit_weighted_sum_and_caps():
    ops = _ops()
    g = torch.Generator().manual_seed(9)
    gu = torch.randn(13, 2 * 37, generator=g) * 3.0
    got = ops.clamped_glu(gu.to(DEV), 1.5, 1.702).cpu().double()
    gate, up = gu[:, :37].double().clamp(max=1.5), gu[:, 37:].double().clamp(-1.5, 1.5)
    assert torch.allclose(got, gate * torch.sigmoid(1.702 * gate) * (up + 1.0), atol=1e-6)
    gu16 = (torch.randn(9, 2 * 48, generator=g) * 3.0).to(torch.bfloat16)     # 16-byte form
    got = ops.clamped_glu(gu16.to(DEV), 2.0, 1.702).cpu().double()
    gate, up = gu16[:, :48].double().clamp(max=2.0), gu16[:, 48:].double().clamp(-2.0, 2.0)
    assert torch.allclose(got, gate * torch.sigmoid(1.702 * gate) * (up + 1.0), rtol=1e-2, atol=1e-2)
    x, y = torch.randn(7, 33, generator=g), torch.randn(7, 33, generator=g).to(torch.bfloat16)
    got = ops.weighted_sum(x.to(DEV), 0.8, y.to(DEV), -0.5).cpu().double()
    assert torch.allclose(got, 0.8 * x.double() - 0.5 * y.double(), atol=1e-6)
    # stacks of partial sums on either side, added in order (and rounded once when asked)
    xs, ys = torch.randn(3, 7, 33, generator=g), torch.randn(5, 7, 33, generator=g)
    got = ops.weighted_sum(xs.to(DEV), 1.5, ys.to(DEV), 0.25).cpu().double()
    assert torch.allclose(got, 1.5 * xs.double().sum(0) + 0.25 * ys.double().sum(0), atol=1e-5)
    got = ops.weighted_sum(xs.to(DEV), 1.0, None, round_parts=True).cpu()
    assert torch.equal(got, ((xs[0] + xs[1]) + xs[2]).to(torch.bfloat16).float())
    # a float32 result from bfloat16 operands at every row count's kernel
    w = (torch.randn(96, 512, generator=g) * 0.05).to(torch.bfloat16)
    for rows in (1, 16, 17, 40, 64, 65, 200):
        xr = torch.randn(rows, 512, generator=g).to(torch.bfloat16)
        got = ops.linear_f32(xr.to(DEV), w.to(DEV)).cpu()
        assert got.dtype == torch.float32 and got.shape == (rows, 96)
        assert torch.allclose(got.double(), xr.double() @ w.double().T, rtol=1e-4, atol=1e-4)
    z = torch.randn(5, 19, generator=g) * 40.0
    assert torch.allclose(ops.soft_cap_(z.clone().to(DEV), 30.0).cpu().double(),
                          30.0 * torch.tanh(z.double() / 30.0), atol=1e-5)


def test_embedding_multiplier_offset_norm_and_residual_multiplier():
    ops = _ops()
    g = torch.Generator().manual_seed(10)
    table = torch.randn(50, 40, generator=g)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    got = ops.embed(ids.to(DEV), table.to(DEV), 16.0).cpu()
    assert torch.equal(got, table[ids.long()] * 16.0)
    for H in (40, 1500, 5000):                         # every row form of the norm kernel
        resid = torch.randn(6, H, generator=g)
        delta = torch.randn(6, H, generator=g)
        w = torch.randn(H, generator=g) * 0.3
        for delta_dtype in (torch.float32, torch.bfloat16):
            d = delta.to(delta_dtype)
            r = resid.clone().to(DEV)
            y = ops.add_rmsnorm(r, d.to(DEV), (w + 1.0).to(DEV), 1e-5, torch.float32,
                                delta_scale=0.7).cpu().double()
            total = resid.double() + 0.7 * d.double()
            assert torch.allclose(r.cpu().double(), total, atol=1e-6)
            assert torch.allclose(y, plain.offset_norm(total, w.double(), 1e-5), atol=1e-5)
            r = resid.clone().to(DEV)
            ops.add_residual(r, d.to(DEV), delta_scale=0.7)
            assert torch.allclose(r.cpu().double(), total, atol=1e-6)
