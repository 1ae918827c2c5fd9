"""The kernels of the Pisulorn design alone, each against the plain function of its mechanism
(tests/plain/pisulorn_plain.py), at sizes that are no power of two and differ from one another.

Like tests/test_kernels_gpu.py these run without a GPU when the environment says RI_TEST_KERNELS=emulated
(tests/test_kernels_emulated.py starts that run): the CPU build of the same sources between guard pages."""
import os

import numpy as np
import pytest
import torch

from plain import pisulorn_plain as P

EMULATED = os.environ.get("RI_TEST_KERNELS") == "emulated"
pytestmark = [] if EMULATED else pytest.mark.gpu
DEV = "cpu" if EMULATED else "cuda:0"
PAGE = 32


@pytest.fixture(scope="module")
def ops():
    if EMULATED:
        import emulated
        return emulated.ops()
    from rust_inference_amd.kernels import ops
    return ops


@pytest.fixture(autouse=True)
def _guarded_buffers_go_back():
    yield
    if EMULATED:
        import gc
        import emulated
        gc.collect()
        emulated.free_all()


def guarded(x):
    if EMULATED:
        import emulated
        return emulated.tensor(x.contiguous(), "a test's operand")
    return x


def t(a, dtype=torch.float32):
    return guarded(torch.tensor(np.asarray(a), dtype=dtype, device=DEV))


def f64(x):
    return x.detach().to("cpu", torch.float64).numpy()


def close(got, want, rel, what=""):
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(f64(got) - want).max() / max(np.abs(want).max(), 1e-30)
    assert err <= rel, f"{what}: error {err:.3e} of the largest value exceeds {rel:.0e}"


F32 = 3e-6
BF16_OUT = 7.5e-3


# ---------------------------------------------------------------- activation
@pytest.mark.parametrize("dtype, n", [(torch.float32, 1001), (torch.bfloat16, 1001), (torch.bfloat16, 2048)])
def test_gelu_tanh(ops, dtype, n):
    x = torch.linspace(-9, 9, n).to(dtype)
    got = ops.gelu_tanh(guarded(x.to(DEV)))
    close(got, P.gelu_tanh(x.to(torch.float64).numpy()), F32 if dtype == torch.float32 else BF16_OUT)


# ---------------------------------------------------------------- attention with a distance bias and a window
def paged(ops, k, v, order, dtype):
    """Keys ``[T, G, dim]`` and values ``[T, G, vdim]`` of one sequence in pages handed out in ``order``."""
    T, G, dim = k.shape
    vdim = v.shape[2]
    pages = -(-T // PAGE)
    kp = torch.zeros((len(order), G, PAGE, dim), dtype=dtype)
    vp = torch.zeros((len(order), G, vdim, PAGE), dtype=dtype)
    for j in range(T):
        kp[order[j // PAGE], :, j % PAGE] = torch.tensor(k[j]).to(dtype)
        vp[order[j // PAGE], :, :, j % PAGE] = torch.tensor(v[j]).to(dtype)
    table = torch.tensor([list(order[:pages]) + [-1] * 2], dtype=torch.int32)
    return guarded(kp.to(DEV)), guarded(vp.to(DEV)), guarded(table.to(DEV))


def bf16_round(a):
    return torch.tensor(a).to(torch.bfloat16).to(torch.float64).numpy()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, kv, dim, vdim, window, T", [(6, 2, 24, 24, 7, 75), (3, 3, 16, 40, None, 70), (4, 1, 64, 64, 33, 300),
                                                            (2, 2, 20, 12, 1, 40)])
def test_generic_attention_with_slopes_and_window(ops, dtype, heads, kv, dim, vdim, window, T):
    rng = np.random.default_rng(heads * 10 + dim)
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": 0.31}
    if window:
        m["mask"] = {"size": window}
    q, k, v = rng.normal(size=(T, heads, dim)), rng.normal(size=(T, kv, dim)), rng.normal(size=(T, kv, vdim))
    if dtype == torch.bfloat16:
        q, k, v = bf16_round(q), bf16_round(k), bf16_round(v)
    new = list(range(T - 9, T)) + [0, window or 3] if T > 60 else list(range(T))      # the last tokens and two early ones
    new = sorted(set(new))
    want = P.attention_core(m, q[new], k, v, new)
    order = list(rng.permutation(-(-T // PAGE) + 2))
    kp, vp, table = paged(ops, k, v, order, dtype)
    qkv = t(q[new].reshape(len(new), -1), dtype)
    got = ops.attention(qkv, kp, vp, t(new, torch.int32), t([0] * len(new), torch.int32), table, heads, kv, dim,
                        window, m["scale"], None, t(P.distance_slopes(heads)))
    close(got, want.reshape(len(new), -1), F32 if dtype == torch.float32 else BF16_OUT)


def test_a_slope_makes_a_near_key_beat_a_far_one(ops):
    """Two keys with the same product with the query, 50 positions apart: with the bias the near one has all the weight."""
    heads, dim, T = 2, 8, 60
    q = np.zeros((1, heads, dim)); q[..., 0] = 4.0
    k = np.zeros((T, 1, dim)); k[5, 0, 0] = k[55, 0, 0] = 3.0
    v = np.zeros((T, 1, dim)); v[5, 0, 0] = 1.0; v[55, 0, 1] = 1.0
    m = {"heads": heads, "kv_heads": 1, "dim": dim, "vdim": dim, "scale": 1.0}
    want = P.attention_core(m, q, k, v, [T - 1])
    assert want[0, 0, 1] > 0.9 * (want[0, 0, 0] + want[0, 0, 1]) and want[0, 0, 0] > 0        # head 0: the slope is 1/16
    kp, vp, table = paged(ops, k, v, list(range(2)), torch.float32)
    got = ops.attention(t(q.reshape(1, -1)), kp, vp, t([T - 1], torch.int32), t([0], torch.int32), table, heads, 1, dim, None,
                        1.0, None, t(P.distance_slopes(heads)))
    close(got, want.reshape(1, -1), F32)


# ---------------------------------------------------------------- the gated delta rule
def delta_case(rng, T, H, G, dk, dv, K):
    C = 2 * G * dk + H * dv
    return dict(proj=rng.normal(size=(T, C + H * dv)), taps=rng.normal(size=(C, K)) * 0.6, ab=rng.normal(size=(T, 2 * H)) * 2,
                a_log=rng.normal(size=H) * 0.5, dt_bias=rng.normal(size=H), C=C)


def plain_prepare(c, H, G, dk, dv, K, lens, tails):
    """q, k, v and the gates of all tokens by the plain functions, sequence by sequence; ``tails`` is changed."""
    qkv, gates, at = [], [], 0
    for b, n in enumerate(lens):
        x = c["proj"][at:at + n, :c["C"]]
        y, tails[b] = P.short_convolution(x, c["taps"], tails[b])
        q = P.unit(y[:, :G * dk].reshape(n, G, dk)) * dk ** -0.5
        k = P.unit(y[:, G * dk:2 * G * dk].reshape(n, G, dk))
        qkv.append(np.concatenate([q.reshape(n, -1), k.reshape(n, -1), y[:, 2 * G * dk:]], 1))
        a, bb = c["ab"][at:at + n, :H], c["ab"][at:at + n, H:]
        gates.append(np.concatenate([np.exp(-np.exp(c["a_log"]) * P.softplus(a + c["dt_bias"])), P.sigmoid(bb)], 1))
        at += n
    return np.concatenate(qkv), np.concatenate(gates)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, dk, dv, K, lens", [(4, 2, 12, 20, 4, (1, 7, 3)), (2, 1, 64, 48, 3, (40,)), (3, 3, 5, 70, 2, (2, 2)),
                                                   (2, 2, 8, 8, 1, (5, 1)), (1, 1, 9, 4, 7, (3, 1, 9))])
def test_delta_prepare_and_the_convolutions_tails(ops, dtype, H, G, dk, dv, K, lens):
    rng = np.random.default_rng(H * 7 + dk)
    T = sum(lens)
    c = delta_case(rng, T, H, G, dk, dv, K)
    if dtype == torch.bfloat16:
        c["proj"] = bf16_round(c["proj"])
    slots = [3, 0, 4][:len(lens)]
    tails = rng.normal(size=(5, K - 1, c["C"]))
    plain_tails = [tails[s].copy() for s in slots]
    want_qkv, want_gates = plain_prepare(c, H, G, dk, dv, K, lens, plain_tails)
    cu = np.concatenate([[0], np.cumsum(lens)])
    seq = np.repeat(np.arange(len(lens)), lens)
    dev_tails = t(tails)
    qkv, gates = ops.delta_prepare(t(c["proj"], dtype), 0, t(c["taps"]), dev_tails, t(c["ab"]), t(c["a_log"]), t(c["dt_bias"]),
                                   t(seq, torch.int32), t(cu, torch.int32), t(slots, torch.int32), H, G, dk, dv)
    close(qkv, want_qkv, F32, "q, k, v")
    close(gates, want_gates, F32, "gates")
    for s, want in zip(slots, plain_tails):
        if K > 1:
            close(dev_tails[s], want, 1e-7, "tail")
    untouched = [s for s in range(5) if s not in slots]
    assert np.array_equal(f64(dev_tails[untouched]), tails[untouched].astype(np.float32).astype(np.float64))


@pytest.mark.parametrize("H, G, dk, dv, lens", [(4, 2, 12, 20, (1, 7, 3)), (2, 1, 64, 48, (45,)), (3, 3, 5, 70, (2, 18)),
                                                (1, 1, 100, 130, (20,)), (2, 2, 33, 8, (17, 1)), (1, 1, 130, 16, (9,)),
                                                (1, 1, 256, 8, (11,))])
@pytest.mark.parametrize("slices", [0, 4, 8])
def test_delta_scan(ops, H, G, dk, dv, lens, slices):
    rng = np.random.default_rng(H * 11 + dk)
    T = sum(lens)
    C = 2 * G * dk + H * dv
    q = P.unit(rng.normal(size=(T, G, dk))) * dk ** -0.5
    k = P.unit(rng.normal(size=(T, G, dk)))
    v = rng.normal(size=(T, H, dv))
    g, beta = rng.uniform(0.3, 1.0, size=(T, H)), rng.uniform(0.1, 1.0, size=(T, H))
    slots = [2, 0, 3][:len(lens)]
    state = rng.normal(size=(4, H, dk, dv))
    want_state, want, at = state.copy(), np.zeros((T, H, dv)), 0
    for b, n in enumerate(lens):
        for h in range(H):
            hq = h // (H // G)
            want[at:at + n, h] = P.delta_recurrence(q[at:at + n, hq], k[at:at + n, hq], v[at:at + n, h], beta[at:at + n, h],
                                                    g[at:at + n, h], want_state[slots[b], h])
        at += n
    qkv = np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1)
    assert qkv.shape[1] == C
    cu = np.concatenate([[0], np.cumsum(lens)])
    dev_state = t(state)
    got = ops.delta_scan(t(qkv), t(np.concatenate([g, beta], 1)), dev_state, t(cu, torch.int32), t(slots, torch.int32), H, G, dk, dv,
                         slices)
    close(got, want.reshape(T, -1), 1e-5, "outputs")
    close(dev_state, want_state, 1e-5, "state")


@pytest.mark.parametrize("slices", [4, 8])
def test_delta_scan_token_by_token_is_the_walk_in_blocks(ops, slices):
    """The same 37 tokens in one step, and one at a time from the state the step before left: the same bits."""
    rng = np.random.default_rng(5)
    H, G, dk, dv, T = 2, 1, 24, 40, 37
    q, k = P.unit(rng.normal(size=(T, G, dk))) * dk ** -0.5, P.unit(rng.normal(size=(T, G, dk)))
    qkv = np.concatenate([q.reshape(T, -1), k.reshape(T, -1), rng.normal(size=(T, H * dv))], 1)
    gates = np.concatenate([rng.uniform(0.3, 1.0, size=(T, H)), rng.uniform(0.1, 1.0, size=(T, H))], 1)
    one, slot = t(np.zeros((2, H, dk, dv))), t([1], torch.int32)
    whole = ops.delta_scan(t(qkv), t(gates), one, t([0, T], torch.int32), slot, H, G, dk, dv, slices)
    two = t(np.zeros((2, H, dk, dv)))
    rows = [ops.delta_scan(t(qkv[i:i + 1]), t(gates[i:i + 1]), two, t([0, 1], torch.int32), slot, H, G, dk, dv, slices) for i in range(T)]
    assert torch.equal(torch.cat([r.cpu() for r in rows]), whole.cpu()) and torch.equal(one.cpu(), two.cpu())


# ---------------------------------------------------------------- mixture of experts
@pytest.mark.parametrize("E, top, T", [(10, 3, 50), (5, 5, 3), (16, 1, 9), (70, 4, 65)])
def test_router(ops, E, top, T):
    rng = np.random.default_rng(E)
    z, corr = rng.normal(size=(T, E)) * 2, rng.normal(size=E) * 0.3
    z32 = z.astype(np.float32).astype(np.float64)
    mlp = {"router": {"experts": E, "top": top}}
    chosen, weights = P.route(mlp, {"r.router": np.eye(E), "r.correction": corr.astype(np.float32).astype(np.float64)}, "r.", z32)
    ids, w, dense = ops.experts_route(t(z), t(corr), top)
    assert np.array_equal(f64(ids).astype(int), chosen)
    close(w, weights, F32)
    want_dense = np.zeros((T, E))
    np.put_along_axis(want_dense, chosen, weights, -1)
    close(dense, want_dense, F32)


def test_the_correction_chooses_and_does_not_weigh(ops):
    """Expert 2 has the lowest score and a large correction: it is chosen, with its small score as its weight."""
    z = np.array([[2.0, 1.0, -3.0, 0.5]])
    corr = np.array([0.0, 0.0, 5.0, 0.0])
    ids, w, dense = ops.experts_route(t(z), t(corr), 2)
    assert f64(ids).astype(int).tolist() == [[2, 0]]
    s = P.sigmoid(z[0])
    close(w, [[s[2] / (s[2] + s[0]), s[0] / (s[2] + s[0])]], F32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_experts_activation(ops, dtype):
    rng = np.random.default_rng(3)
    T, E, ff, limit = 6, 5, 13, 0.8
    gu = rng.normal(size=(T, E, 2, ff)) * 1.5
    if dtype == torch.bfloat16:
        gu = bf16_round(gu)
    dense = rng.uniform(0.1, 1, size=(T, E)) * (rng.uniform(size=(T, E)) < 0.5)
    g, u = np.minimum(gu[:, :, 0], limit), np.clip(gu[:, :, 1], -limit, limit)
    want = dense[:, :, None] * (g * P.sigmoid(1.702 * g) * (u + 1.0))
    got = ops.experts_activate(t(gu.reshape(T, -1), dtype), t(dense), ff, limit)
    close(got, want.reshape(T, -1), F32 if dtype == torch.float32 else BF16_OUT)
    assert (f64(got).reshape(T, E, ff)[dense == 0] == 0).all()


# ---------------------------------------------------------------- the distance bias on the matrix cores
def paged_batch(ops, k, v, lens, seed):
    """Keys and values of several sequences (flat, one after the other) in pages handed out in shuffled order."""
    G, dk, dv = k.shape[1], k.shape[2], v.shape[2]
    width = max(-(-n // PAGE) for n in lens) + 1
    n_pages = sum(-(-n // PAGE) for n in lens) + 2
    order = np.random.default_rng(seed).permutation(n_pages)
    table = np.full((len(lens), width), -1, dtype=np.int32)
    kp = torch.zeros((n_pages, G, PAGE, dk), dtype=torch.bfloat16)
    vp = torch.zeros((n_pages, G, dv, PAGE), dtype=torch.bfloat16)
    nxt = at = 0
    for b, n in enumerate(lens):
        for p in range(-(-n // PAGE)):
            table[b, p] = order[nxt]
            nxt += 1
        for j in range(n):
            kp[table[b, j // PAGE], :, j % PAGE] = torch.tensor(k[at + j]).bfloat16()
            vp[table[b, j // PAGE], :, :, j % PAGE] = torch.tensor(v[at + j]).bfloat16()
        at += n
    return guarded(kp.to(DEV)), guarded(vp.to(DEV)), t(table, torch.int32)


@pytest.mark.parametrize("form", ["prefill", "decode"])
@pytest.mark.parametrize("dh, heads, kv_heads, window", [(64, 8, 4, 41), (128, 4, 1, None), (32, 2, 2, 33), (64, 6, 3, 100), (64, 16, 1, 7)])
def test_the_matrix_core_kernels_take_the_distance_bias(ops, form, dh, heads, kv_heads, window):
    """bfloat16, heads of 32, 64 and 128, with and without a window: prompts of unequal lengths, and one new token each
    after them; scores small enough for the bias to decide most weights."""
    rng = np.random.default_rng(dh + heads)
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dh, "vdim": dh, "scale": 0.05}
    if window:
        m["mask"] = {"size": window}
    lens = [75, 1, 40] if form == "prefill" else [300, 33, 64]
    T = sum(lens)
    q, k, v = (bf16_round(rng.normal(size=(T, heads, dh))), bf16_round(rng.normal(size=(T, kv_heads, dh))),
               bf16_round(rng.normal(size=(T, kv_heads, dh))))
    kp, vp, table = paged_batch(ops, k, v, lens, dh)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tok_pos = np.concatenate([np.arange(n) for n in lens])
    tok_seq = np.repeat(np.arange(len(lens)), lens)
    want = np.concatenate([P.attention_core(m, q[a:b], k[a:b], v[a:b], np.arange(b - a)).reshape(b - a, -1)
                           for a, b in zip(cu[:-1], cu[1:])])
    slopes = t(P.distance_slopes(heads))
    qkv = t(q.reshape(T, -1), torch.bfloat16)
    if form == "prefill":
        got = ops.attention_prefill_bf16(qkv, kp, vp, t(cu, torch.int32), t(tok_pos, torch.int32), table, len(lens), max(lens),
                                         heads, kv_heads, dh, window, m["scale"], None, slopes)
        close(got, want, BF16_OUT, "prefill")
    else:
        last = cu[1:] - 1                                      # each sequence's last token as its one new token
        rows = t(q[last].reshape(len(lens), -1), torch.bfloat16)
        got = ops.attention_decode_bf16(rows, kp, vp, t(np.arange(len(lens) + 1), torch.int32),
                                        t([n - 1 for n in lens], torch.int32), table, len(lens), max(lens), heads, kv_heads,
                                        dh, window, m["scale"], slopes=slopes)
        close(got, want[last], BF16_OUT, "decode")
    same = ops.attention(qkv, kp, vp, t(tok_pos, torch.int32), t(tok_seq, torch.int32), table, heads, kv_heads, dh, window,
                         m["scale"], None, slopes)
    close(same, want, BF16_OUT, "the generic kernel on the same pages")


def test_the_matrix_core_kernels_weigh_two_equal_keys_by_their_distance(ops):
    """Two keys with the same large product with the last query, 1,200 and 3 positions back: without the bias they
    share the weight, with it the near one has it all, for the one-token kernels and the prompt kernel alike."""
    rng = np.random.default_rng(4)
    n, dh, heads = 1300, 64, 2
    m = {"heads": heads, "kv_heads": 1, "dim": dh, "vdim": dh, "scale": 1.0}
    k, v, q = rng.normal(size=(n, 1, dh)) * 0.1, rng.normal(size=(n, 1, dh)), rng.normal(size=(n, heads, dh)) * 0.1
    for j in (n - 1 - 1200, n - 1 - 3):
        k[j, 0] = 0.0
        k[j, 0, 9] = 6.0
    q[-1] = 0.0
    q[-1, :, 9] = 6.0
    q, k, v = bf16_round(q), bf16_round(k), bf16_round(v)
    kp, vp, table = paged_batch(ops, k, v, [n], 1)
    want = P.attention_core(m, q, k, v, np.arange(n)).reshape(n, -1)
    near = v[n - 1 - 3, 0]
    assert np.abs(want[-1, :dh] - near).max() < 1e-3            # head 0's slope is 1/16: 1,197 positions are 75 in the exponent
    slopes = t(P.distance_slopes(heads))
    qkv = t(q.reshape(n, -1), torch.bfloat16)
    whole = ops.attention_prefill_bf16(qkv, kp, vp, t([0, n], torch.int32), t(np.arange(n), torch.int32), table, 1, n, heads, 1,
                                       dh, None, 1.0, None, slopes)
    last = ops.attention_decode_bf16(t(q[-1:].reshape(1, -1), torch.bfloat16), kp, vp, t([0, 1], torch.int32),
                                     t([n - 1], torch.int32), table, 1, n, heads, 1, dh, None, 1.0, slopes=slopes)
    close(whole, want, BF16_OUT, "prompt")
    close(last, want[-1:], BF16_OUT, "one token")
    plain = ops.attention_decode_bf16(t(q[-1:].reshape(1, -1), torch.bfloat16), kp, vp, t([0, 1], torch.int32),
                                      t([n - 1], torch.int32), table, 1, n, heads, 1, dh, None, 1.0)
    assert np.abs(f64(plain)[0, :dh] - near).max() > 0.1         # without slopes the far key has half the weight


# ---------------------------------------------------------------- the experts of a few tokens, and of many
def experts_case(rng, T, E, top, ff, dim, limit):
    x = bf16_round(rng.normal(size=(T, dim)))
    w = {"m.router": bf16_round(rng.normal(size=(E, dim)) * 0.3), "m.correction": rng.normal(size=E) * 0.2}
    for e in range(E):
        w[f"m.e{e}.gate"] = bf16_round(rng.normal(size=(ff, dim)) * 0.2)
        w[f"m.e{e}.up"] = bf16_round(rng.normal(size=(ff, dim)) * 0.2)
        w[f"m.e{e}.down"] = bf16_round(rng.normal(size=(dim, ff)) * 0.2)
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": E, "top": top}}
    gate_up = np.concatenate([np.concatenate([w[f"m.e{e}.gate"], w[f"m.e{e}.up"]]) for e in range(E)])
    down = np.concatenate([w[f"m.e{e}.down"] for e in range(E)], 1)
    return x, w, mlp, gate_up, down


@pytest.mark.parametrize("T, E, top, ff, dim", [(1, 7, 3, 24, 40), (5, 4, 1, 520, 72), (8, 6, 5, 16, 1032), (3, 3, 2, 8, 8)])
def test_the_experts_of_a_few_tokens(ops, T, E, top, ff, dim):
    rng = np.random.default_rng(T + E)
    x, w, mlp, gate_up, down = experts_case(rng, T, E, top, ff, dim, 0.9)
    want = P.moe_ff(mlp, w, "m.", x)
    ids, weights, _ = ops.experts_route(t(x @ w["m.router"].T), t(w["m.correction"]), top)
    got = ops.experts_few_tokens(t(x, torch.bfloat16), t(gate_up, torch.bfloat16), t(down, torch.bfloat16), ids, weights, ff, 0.9)
    close(got, want, BF16_OUT)


@pytest.mark.parametrize("T, E, top, dim", [(300, 7, 3, 40), (70, 5, 1, 16), (9, 3, 3, 8), (1, 70, 4, 24), (520, 2, 1, 8), (5, 4, 2, 2056)])
def test_the_assignments_sorted_by_expert(ops, T, E, top, dim):
    rng = np.random.default_rng(T)
    ids = np.stack([rng.permutation(E)[:top] for _ in range(T)]).astype(np.int32)
    dest, offsets = ops.experts_sort(t(ids, torch.int32), E)
    flat = ids.reshape(-1)
    order = np.argsort(flat, kind="stable")                   # by expert, inside an expert by token
    want_dest = np.empty_like(order)
    want_dest[order] = np.arange(len(order))
    assert np.array_equal(f64(dest).astype(int), want_dest)
    assert np.array_equal(f64(offsets).astype(int), np.concatenate([[0], np.cumsum(np.bincount(flat, minlength=E))]))
    x = bf16_round(rng.normal(size=(T, dim)))
    rows = ops.experts_gather(t(x, torch.bfloat16), dest, top)
    assert np.array_equal(f64(rows)[want_dest], np.repeat(x, top, 0))
    weights = rng.uniform(0.1, 1, size=(T, top))
    y = bf16_round(rng.normal(size=(T * top, dim)))
    got = ops.experts_combine(t(y, torch.bfloat16), dest, t(weights))
    close(got, (weights[:, :, None] * y[want_dest].reshape(T, top, dim)).sum(1), F32)


def test_the_weighted_sum_of_rows_of_an_odd_size(ops):
    rng = np.random.default_rng(2)
    T, top, dim = 6, 3, 21
    dest = rng.permutation(T * top).astype(np.int32)
    y, weights = bf16_round(rng.normal(size=(T * top, dim))), rng.uniform(0.1, 1, size=(T, top))
    got = ops.experts_combine(t(y, torch.bfloat16), t(dest, torch.int32), t(weights))
    close(got, (weights[:, :, None] * y[dest].reshape(T, top, dim)).sum(1), F32)


def test_an_experts_rows_activated_without_weights(ops):
    rng = np.random.default_rng(8)
    gu = rng.normal(size=(7, 2, 20)) * 2
    g, u = np.minimum(gu[:, 0], 1.1), np.clip(gu[:, 1], -1.1, 1.1)
    got = ops.experts_activate(t(gu.reshape(7, -1)), None, 20, 1.1)
    close(got, g * P.sigmoid(1.702 * g) * (u + 1.0), F32)


# ---------------------------------------------------------------- the delta rule's one-token kernel
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, G, dk, dv, K", [(4, 2, 12, 20, 4), (2, 1, 64, 48, 3), (3, 3, 5, 72, 2), (2, 2, 128, 128, 4),
                                             (1, 1, 60, 132, 1), (2, 1, 256, 40, 5), (1, 1, 9, 256, 2), (2, 2, 33, 4, 3)])
def test_delta_step_of_one_token_a_sequence(ops, dtype, H, G, dk, dv, K):
    """Against the plain functions, and against the kernels of the prompt path on the same inputs: states that are not
    zero, on slots in another order, tails partly filled."""
    assert ops.delta_step_fits(dk, dv)
    rng = np.random.default_rng(H * 13 + dv)
    B = 3
    c = delta_case(rng, B, H, G, dk, dv, K)
    if dtype == torch.bfloat16:
        c["proj"] = bf16_round(c["proj"])
    slots = [3, 0, 4]
    tails, state, gain = rng.normal(size=(5, K - 1, c["C"])), rng.normal(size=(5, H, dk, dv)) * 0.3, 1 + 0.1 * rng.normal(size=dv)
    plain_tails = [tails[s].copy() for s in slots]
    qkv, gates = plain_prepare(c, H, G, dk, dv, K, [1] * B, plain_tails)
    want_state, want = state.copy(), np.zeros((B, H, dv))
    for b in range(B):
        for h in range(H):
            hq = h // (H // G)
            o = P.delta_recurrence(qkv[b:b + 1, hq * dk:(hq + 1) * dk], qkv[b:b + 1, (G + hq) * dk:(G + hq + 1) * dk],
                                   qkv[b:b + 1, 2 * G * dk + h * dv:2 * G * dk + (h + 1) * dv], gates[b:b + 1, H + h],
                                   gates[b:b + 1, h], want_state[slots[b], h])
            want[b, h] = P.rms_norm(o[0], gain, 1e-5) * P.silu(c["proj"][b, c["C"] + h * dv:c["C"] + (h + 1) * dv])
    dev_tails, dev_state = t(tails), t(state)
    got = ops.delta_step(t(c["proj"], dtype), 0, c["C"], t(c["taps"]), dev_tails, t(c["ab"]), t(c["a_log"]), t(c["dt_bias"]),
                         dev_state, t(np.arange(B + 1), torch.int32), t(slots, torch.int32), t(gain), 1e-5, H, G, dk, dv)
    close(got, want.reshape(B, -1), 2e-5 if dtype == torch.float32 else BF16_OUT, "outputs")
    close(dev_state, want_state, 1e-5, "state")
    for s, w in zip(slots, plain_tails):
        if K > 1:
            close(dev_tails[s], w, 1e-7, "tail")


def test_delta_step_does_not_fit_every_size(ops):
    assert not ops.delta_step_fits(300, 64) and not ops.delta_step_fits(64, 300) and not ops.delta_step_fits(64, 70)
    assert not ops.delta_step_fits(128, 256) and ops.delta_step_fits(256, 64) and ops.delta_step_fits(64, 256)


def test_many_sequences_take_the_streaming_kernel_with_the_distance_bias(ops):
    """64 sequences of 8 kv heads are the 512 pairs from which a decode step walks whole runs of pages a workgroup:
    that kernel too takes the slopes and the window."""
    rng = np.random.default_rng(12)
    dh, heads, kv_heads, window = 64, 16, 8, 50
    lens = [int(n) for n in rng.integers(3, 150, 64)]
    assert ops.decode_attention_streams(len(lens), kv_heads, max(lens))
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dh, "vdim": dh, "scale": 0.07, "mask": {"size": window}}
    T = sum(lens)
    k, v = bf16_round(rng.normal(size=(T, kv_heads, dh))), bf16_round(rng.normal(size=(T, kv_heads, dh)))
    cu = np.concatenate([[0], np.cumsum(lens)])
    q = bf16_round(rng.normal(size=(len(lens), heads, dh)))        # each sequence's last token is its one new token
    want = np.stack([P.attention_core(m, q[b:b + 1], k[cu[b]:cu[b + 1]], v[cu[b]:cu[b + 1]], [lens[b] - 1]).reshape(-1)
                     for b in range(len(lens))])
    kp, vp, table = paged_batch(ops, k, v, lens, 3)
    got = ops.attention_decode_bf16(t(q.reshape(len(lens), -1), torch.bfloat16), kp, vp, t(np.arange(len(lens) + 1), torch.int32),
                                    t([n - 1 for n in lens], torch.int32), table, len(lens), max(lens), heads, kv_heads, dh, window,
                                    m["scale"], slopes=t(P.distance_slopes(heads)))
    close(got, want, BF16_OUT)
