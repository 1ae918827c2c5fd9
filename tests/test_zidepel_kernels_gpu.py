"""The kernels of the Zidepel design alone, each against the plain function of its mechanism
(tests/plain/zidepel_plain.py), at sizes that are no power of two and differ from one another.

Like tests/test_kernels_gpu.py these run without a GPU when the environment says RI_TEST_KERNELS=emulated
(tests/test_kernels_emulated.py starts that run): the CPU build of the same sources between guard pages."""
import os

import numpy as np
import pytest
import torch

from plain import zidepel_plain as Z

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


F32 = 2e-6
BF16_OUT = 7.5e-3


# ---------------------------------------------------------------- streams and norms
@pytest.mark.parametrize("streams, dim", [(4, 104), (1, 200), (3, 72), (8, 40), (2, 70), (16, 33), (4, 5000)])
@pytest.mark.parametrize("kind", ["layer", "rms", "none"])
def test_streams_write_read_and_norm(ops, streams, dim, kind):
    rng = np.random.default_rng(streams * 100 + dim)
    T = 5
    x = rng.normal(size=(T, streams, dim))
    y = rng.normal(size=(T, dim))
    mix, outw, inw = rng.normal(size=(streams, streams)), rng.normal(size=streams), rng.normal(size=streams)
    gain, bias = rng.normal(size=dim), rng.normal(size=dim)
    eps = 1e-3
    # the plain form works on [S, T, dim] with w[prefix + ...]
    w = {"p.in": inw, "p.mix": mix, "p.out": outw}
    new = Z.hyper_sublayer(x.transpose(1, 0, 2), {**w, "p.in": np.zeros(streams)}, "p.", lambda u: y)     # the write alone
    u = np.tensordot(inw, new, axes=(0, 0))
    want = {"layer": Z.layer_norm(u, gain, bias, eps), "rms": Z.rms_norm(u, gain, eps), "none": u}[kind]
    code = {"layer": ops.NORM_LAYER, "rms": ops.NORM_RMS, "none": ops.NORM_NONE}[kind]
    xs = t(x)
    got = ops.streams_read_norm(xs, t(y), t(mix), t(outw), t(inw), t(gain), t(bias) if kind == "layer" else None, eps,
                                code, torch.float32)
    close(got, want, F32, "normed read")
    close(xs, new.transpose(1, 0, 2), F32, "streams after the write")
    # gathered rows: nothing is stored
    xs2 = t(x)
    rows = t([3, 0, 3], torch.int32)
    got = ops.streams_read_norm(xs2, t(y), t(mix), t(outw), t(inw), t(gain), t(bias) if kind == "layer" else None, eps,
                                code, torch.float32, rows=rows)
    close(got, want[[3, 0, 3]], F32, "gathered rows")
    assert np.array_equal(f64(xs2), x.astype(np.float32).astype(np.float64))
    # pending in bfloat16 and in parts
    yb = torch.tensor(y, dtype=torch.bfloat16)
    parts = rng.normal(size=(3, T, dim))
    for pend, yy in ((t(f64(yb), torch.bfloat16), f64(yb)), (t(parts), parts.astype(np.float32).astype(np.float64).sum(0))):
        new = Z.hyper_sublayer(x.transpose(1, 0, 2), {**w, "p.in": np.zeros(streams)}, "p.", lambda u: yy)
        xs3 = t(x)
        ops.streams_read_norm(xs3, pend, t(mix), t(outw), t(inw), t(gain), None, eps, ops.NORM_RMS, torch.bfloat16)
        close(xs3, new.transpose(1, 0, 2), F32, "streams after a bfloat16 or split write")


def test_streams_start_from_one_row_and_the_plain_residual_is_one_stream(ops):
    rng = np.random.default_rng(5)
    T, S, dim = 4, 4, 88
    x0 = rng.normal(size=(T, dim))
    inw, gain, bias = rng.normal(size=S), rng.normal(size=dim), rng.normal(size=dim)
    xs = t(np.full((T, S, dim), 7.0))
    got = ops.streams_read_norm(xs, None, None, None, t(inw), t(gain), t(bias), 1e-5, ops.NORM_LAYER, torch.bfloat16,
                                fresh=t(x0))
    close(xs, np.repeat(x0[:, None], S, 1), F32, "spread")
    close(got, Z.layer_norm(inw.sum() * x0, gain, bias, 1e-5), BF16_OUT, "first read")
    # one stream, no coefficients: residual += pending, then the layer norm
    r, y = rng.normal(size=(T, dim)), rng.normal(size=(T, dim))
    res = t(r.reshape(T, 1, dim))
    got = ops.streams_read_norm(res, t(y), None, None, None, t(gain), t(bias), 1e-5, ops.NORM_LAYER, torch.float32)
    close(res.view(T, dim), r + y, F32)
    close(got, Z.layer_norm(r + y, gain, bias, 1e-5), F32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim", [136, 70, 2052])
def test_embedding_with_positions_and_norm(ops, dtype, dim):
    rng = np.random.default_rng(1)
    table, pos = t(rng.normal(size=(300, dim)), dtype), t(rng.normal(size=(50, dim)), dtype)
    gain, bias = rng.normal(size=dim), rng.normal(size=dim)
    ids, where = [299, 0, 7, 7], [0, 49, 3, 4]
    cfg = {"norm": {"eps": 1e-5}}
    w = {"embed": f64(table), "pos": f64(pos), "embed.norm": gain, "embed.norm.b": bias}
    want = np.concatenate([Z.embed(cfg, w, [i], p) for i, p in zip(ids, where)])
    got = ops.embed_positions_norm(table, pos, t(ids, torch.int32), t(where, torch.int32), t(gain), t(bias), 1e-5,
                                   ops.NORM_LAYER)
    close(got, want, F32)


# ---------------------------------------------------------------- attention
def paged(ops, m, q, k, v, lens, dtype, shuffle_seed=0):
    """Runs norm, temperature and cache write, then attention, for sequences of ``lens`` tokens laid out flat;
    pages are handed out in a shuffled order."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = sum(lens)
    width = max(-(-n // PAGE) for n in lens)
    n_pages = sum(-(-n // PAGE) for n in lens) + 2
    order = np.random.default_rng(shuffle_seed).permutation(n_pages)
    table = np.full((len(lens), width), -1, dtype=np.int32)
    nxt = 0
    for b, n in enumerate(lens):
        for p in range(-(-n // PAGE)):
            table[b, p] = order[nxt]
            nxt += 1
    tok_seq = np.concatenate([np.full(n, b) for b, n in enumerate(lens)]).astype(np.int32)
    tok_pos = np.concatenate([np.arange(n) for n in lens]).astype(np.int32)
    qkv = t(np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1), dtype)
    kp = guarded(torch.zeros((n_pages, G, PAGE, dk), dtype=dtype, device=DEV))
    vp = guarded(torch.zeros((n_pages, G, dv, PAGE), dtype=dtype, device=DEV))
    return qkv, kp, vp, t(tok_pos, torch.int32), t(tok_seq, torch.int32), t(table, torch.int32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m", [
    {"heads": 6, "kv_heads": 2, "dim": 24, "vdim": 40, "scale": 0.31, "softcap": 5.0, "q_temp": {"coef": 0.4, "every": 7}},
    {"heads": 3, "kv_heads": 3, "dim": 72, "vdim": 16, "scale": 0.05, "softcap": None, "q_temp": None},
    {"heads": 4, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 1.7, "softcap": 0.8, "q_temp": {"coef": 1.5, "every": 1}},
    {"heads": 4, "kv_heads": 2, "dim": 64, "vdim": 40, "scale": 0.2, "softcap": 9.0, "q_temp": {"coef": 0.3, "every": 16}},
], ids=["capped-tempered", "plain", "one-kv-head", "heads-of-64"])
@pytest.mark.parametrize("by_pages", [False, True], ids=["element-wise", "prompt-kernels"])
def test_norm_temperature_cache_write_and_capped_attention(ops, dtype, m, by_pages):
    rng = np.random.default_rng(3)
    lens = [70, 1, 33]
    T = sum(lens)
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = rng.normal(size=(T, H, dk)) * 2, rng.normal(size=(T, G, dk)) * 2, rng.normal(size=(T, G, dv))
    qg, kg = rng.normal(size=dk), rng.normal(size=dk)
    qkv, kp, vp, tok_pos, tok_seq, table = paged(ops, m, q, k, v, lens, dtype)
    rq, rk, rv = (f64(qkv)[:, :H * dk].reshape(T, H, dk), f64(qkv)[:, H * dk:(H + G) * dk].reshape(T, G, dk),
                  f64(qkv)[:, (H + G) * dk:].reshape(T, G, dv))
    temper = (m["q_temp"]["coef"], m["q_temp"]["every"]) if m["q_temp"] else None
    prompt = dict(cu_seqlens=t(np.concatenate([[0], np.cumsum(lens)]), torch.int32), max_new=max(lens)) if by_pages else {}
    ops.qk_norm_temper_kv_write(qkv, t(qg), t(kg), 1e-5, temper, tok_pos, tok_seq, table, kp, vp, H, G, dk, dv, **prompt)
    got = ops.attention(qkv, kp, vp, tok_pos, tok_seq, table, H, G, dk, None, m["scale"], m["softcap"])
    want, want_q = [], []
    at = 0
    for n in lens:
        pos = np.arange(n)
        qq = Z.rms_norm(rq[at:at + n], qg, 1e-5) * Z.query_temperature(pos, m["q_temp"])[:, None, None]
        kk = Z.rms_norm(rk[at:at + n], kg, 1e-5)
        if dtype == torch.bfloat16:              # what the kernel hands on is rounded once
            qq = f64(torch.tensor(qq).bfloat16())
            kk = f64(torch.tensor(kk).bfloat16())
        want_q.append(qq)
        want.append(Z.attention_core(m, qq, kk, rv[at:at + n], pos).reshape(n, -1))
        at += n
    tol = F32 * 4 if dtype == torch.float32 else BF16_OUT
    close(qkv[:, :H * dk], np.concatenate(want_q).reshape(T, -1), 1e-6 if dtype == torch.float32 else 4e-3, "q in place")    # bfloat16: a last place where float32 and float64 round apart
    close(got, np.concatenate(want), tol, "attention")


def test_one_far_key_is_found_and_the_cap_holds_it_back(ops):
    """A key 900 tokens back whose score stands far out: uncapped the output is its value row; capped at c the
    score is c tanh(s / c), so the other keys keep a share that the plain form gives too."""
    rng = np.random.default_rng(9)
    n, dk, dv = 1000, 32, 24
    m = {"heads": 1, "kv_heads": 1, "dim": dk, "vdim": dv, "scale": 1.0, "softcap": None, "q_temp": None}
    k = rng.normal(size=(n, 1, dk)) * 0.1
    v = rng.normal(size=(n, 1, dv))
    q = rng.normal(size=(n, 1, dk)) * 0.1
    k[97, 0] = 0.0
    k[97, 0, 5] = 6.0
    q[-1, 0] = 0.0
    q[-1, 0, 5] = 6.0
    for cap in (None, 3.0):
        m["softcap"] = cap
        qkv, kp, vp, tok_pos, tok_seq, table = paged(ops, m, q, k, v, [n], torch.float32)
        ops.qk_norm_temper_kv_write(qkv, None, None, 1e-5, None, tok_pos, tok_seq, table, kp, vp, 1, 1, dk, dv)
        got = ops.attention(qkv, kp, vp, tok_pos, tok_seq, table, 1, 1, dk, None, 1.0, cap)
        want = Z.attention_core(m, q.astype(np.float32).astype(np.float64), k.astype(np.float32).astype(np.float64),
                                v.astype(np.float32).astype(np.float64), np.arange(n))[-1, 0]
        close(got[-1], want, 1e-5, f"cap {cap}")
        if cap is None:
            assert np.abs(f64(got[-1]) - v[97, 0]).max() < 1e-4
        else:
            assert np.abs(f64(got[-1]) - v[97, 0]).max() > 0.05


@pytest.mark.parametrize("form", ["prefill", "decode"])
@pytest.mark.parametrize("dh, heads, kv_heads, cap", [(64, 8, 2, 4.0), (128, 4, 1, 11.0), (32, 2, 2, 0.7), (64, 4, 4, None)])
def test_the_matrix_core_kernels_cap_their_scores(ops, form, dh, heads, kv_heads, cap):
    """bfloat16, heads of 32, 64 and 128: prompts of unequal lengths, and one new token each after them, with
    scores large enough for the cap to bend most of them."""
    rng = np.random.default_rng(dh)
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dh, "vdim": dh, "scale": 0.4, "softcap": cap, "q_temp": None}
    lens = [75, 1, 40] if form == "prefill" else [300, 33, 64]
    T = sum(lens)
    q, k, v = rng.normal(size=(T, heads, dh)), rng.normal(size=(T, kv_heads, dh)), rng.normal(size=(T, kv_heads, dh))
    qkv, kp, vp, tok_pos, tok_seq, table = paged(ops, m, q, k, v, lens, torch.bfloat16)
    r = f64(qkv)
    rq, rk, rv = (r[:, :heads * dh].reshape(T, heads, dh), r[:, heads * dh:(heads + kv_heads) * dh].reshape(T, kv_heads, dh),
                  r[:, (heads + kv_heads) * dh:].reshape(T, kv_heads, dh))
    ops.qk_norm_temper_kv_write(qkv, None, None, 1e-5, None, tok_pos, tok_seq, table, kp, vp, heads, kv_heads, dh, dh)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    want = np.concatenate([Z.attention_core(m, rq[a:b], rk[a:b], rv[a:b], np.arange(b - a)).reshape(b - a, -1)
                           for a, b in zip(cu[:-1], cu[1:])])
    if form == "prefill":
        got = ops.attention_prefill_bf16(qkv, kp, vp, t(cu, torch.int32), tok_pos, table, len(lens), max(lens), heads,
                                         kv_heads, dh, None, m["scale"], cap)
        close(got, want, BF16_OUT, "prefill")
    else:
        last = cu[1:] - 1                                      # each sequence's last token as its one new token
        rows = guarded(qkv[torch.tensor(last, dtype=torch.long)].clone())
        got = ops.attention_decode_bf16(rows, kp, vp, t(np.arange(len(lens) + 1), torch.int32),
                                        t([n - 1 for n in lens], torch.int32), table, len(lens), max(lens), heads, kv_heads,
                                        dh, None, m["scale"], softcap=cap)
        close(got, want[last], BF16_OUT, "decode")
    same = ops.attention(qkv, kp, vp, tok_pos, tok_seq, table, heads, kv_heads, dh, None, m["scale"], cap)
    close(same, want, BF16_OUT, "the generic kernel on the same pages")


@pytest.mark.parametrize("cap", [None, 2.5])
def test_the_matrix_core_kernels_find_one_far_key(ops, cap):
    """1,500 keys in bfloat16, the one that matters 1,400 back, behind five chunk borders: the last token alone (the
    one-token kernels) and the whole prompt (the prompt kernel).  Uncapped the output is that key's value row."""
    rng = np.random.default_rng(11)
    n, dh = 1500, 64
    m = {"heads": 2, "kv_heads": 1, "dim": dh, "vdim": dh, "scale": 1.0, "softcap": cap, "q_temp": None}
    k, v, q = rng.normal(size=(n, 1, dh)) * 0.1, rng.normal(size=(n, 1, dh)), rng.normal(size=(n, 2, dh)) * 0.1
    k[97, 0] = 0.0
    k[97, 0, 9] = 6.0
    q[-1] = 0.0
    q[-1, :, 9] = 6.0
    qkv, kp, vp, tok_pos, tok_seq, table = paged(ops, m, q, k, v, [n], torch.bfloat16)
    r = f64(qkv)
    ops.qk_norm_temper_kv_write(qkv, None, None, 1e-5, None, tok_pos, tok_seq, table, kp, vp, 2, 1, dh, dh)
    want = Z.attention_core(m, r[:, :2 * dh].reshape(n, 2, dh), r[:, 2 * dh:3 * dh].reshape(n, 1, dh),
                            r[:, 3 * dh:].reshape(n, 1, dh), np.arange(n)).reshape(n, -1)
    whole = ops.attention_prefill_bf16(qkv, kp, vp, t([0, n], torch.int32), tok_pos, table, 1, n, 2, 1, dh, None, 1.0, cap)
    last = ops.attention_decode_bf16(guarded(qkv[-1:].clone()), kp, vp, t([0, 1], torch.int32), t([n - 1], torch.int32), table,
                                     1, n, 2, 1, dh, None, 1.0, softcap=cap)
    close(whole, want, BF16_OUT, "prompt")
    close(last, want[-1:], BF16_OUT, "one token")
    far = f64(t(v[97, 0], torch.bfloat16))
    if cap is None:
        assert np.abs(f64(last)[0, :dh] - far).max() < 2e-2
    else:
        assert np.abs(f64(last)[0, :dh] - far).max() > 0.1


# ---------------------------------------------------------------- gated linear attention
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, dk, dv, lens", [(3, 24, 40, [19, 1, 8]), (2, 72, 16, [5]), (1, 200, 17, [3, 2]),
                                                  (2, 64, 32, [9, 2]), (1, 128, 16, [20, 1]),
                                                  # enough (sequence, head, column tile) triples for 8 and for 16 columns a workgroup
                                                  (8, 16, 32, [2, 1] * 16), (8, 16, 32, [1, 3] * 32)])
def test_gla_scan_and_output_gate(ops, dtype, heads, dk, dv, lens):
    rng = np.random.default_rng(dk)
    T = sum(lens)
    tau = 3.5
    pad = 8 if dk % 64 == 0 else 5                       # (rows of whole 16-byte pieces take the 16-byte norm and gate)
    proj = t(rng.normal(size=(T, 2 * heads * dk + 2 * heads * dv + pad)), dtype)      # q | k | unused | v | g
    q_off, k_off, v_off = 0, heads * dk, 2 * heads * dk + pad
    g_off = v_off + heads * dv
    z = rng.normal(size=(T, heads * dk)) * 3
    zb = rng.normal(size=heads * dk)
    slots = [4, 0, 2][:len(lens)] if len(lens) <= 3 else list(rng.permutation(len(lens) + 3)[:len(lens)])
    state0 = rng.normal(size=(max(6, len(lens) + 3), heads, dk, dv))
    state = t(state0)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    o = ops.gla_scan(proj, q_off, k_off, v_off, t(z), t(zb), tau, dk ** -0.5, state, t(cu, torch.int32),
                     t(slots, torch.int32), heads, dk, dv)
    p = f64(proj)
    alpha = Z.sigmoid(f64(t(z)) + f64(t(zb))) ** (1.0 / tau)
    want = np.zeros((T, heads, dv))
    want_state = state0.astype(np.float32).astype(np.float64)
    for b, n in enumerate(lens):
        rows = slice(cu[b], cu[b] + n)
        for h in range(heads):
            want[rows, h] = Z.gla_recurrence(p[rows, q_off + h * dk:q_off + (h + 1) * dk] * dk ** -0.5,
                                             p[rows, k_off + h * dk:k_off + (h + 1) * dk],
                                             p[rows, v_off + h * dv:v_off + (h + 1) * dv],
                                             alpha[rows, h * dk:(h + 1) * dk], want_state[slots[b], h])
    close(o, want.reshape(T, -1), 5e-6, "scan")
    close(state, want_state, 5e-6, "state")
    gain = rng.normal(size=dv)
    got = ops.gla_norm_gate(o, proj, g_off, t(gain), 1e-5, heads, dv)
    gate = p[:, g_off:g_off + heads * dv].reshape(T, heads, dv)
    want_out = Z.rms_norm(f64(o).reshape(T, heads, dv), gain, 1e-5) * Z.silu(gate)
    close(got, want_out.reshape(T, -1), F32 * 2 if dtype == torch.float32 else BF16_OUT, "normed and gated")


def test_values_go_into_pages_from_any_start(ops):
    """A prompt's portion that begins in the middle of a page and ends in the middle of another, beside a whole
    page and a single token: the page-wise writer against the element-wise one."""
    rng = np.random.default_rng(4)
    H, G, dk, dv = 2, 2, 16, 24
    starts, counts = [13, 64, 31], [70, 32, 1]
    T = sum(counts)
    width = 4
    table = np.array([[5, 2, 9, 0], [7, 1, 3, 11], [4, 10, 6, 8]], dtype=np.int32)
    tok_seq = np.concatenate([np.full(n, b) for b, n in enumerate(counts)]).astype(np.int32)
    tok_pos = np.concatenate([np.arange(s, s + n) for s, n in zip(starts, counts)]).astype(np.int32)
    cu = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    for dtype in (torch.bfloat16, torch.float32):
        x = rng.normal(size=(T, (H + G) * dk + G * dv))
        pages = []
        for prompt in ({}, dict(cu_seqlens=t(cu, torch.int32), max_new=max(counts))):
            qkv = t(x, dtype)
            kp = guarded(torch.zeros((12, G, PAGE, dk), dtype=dtype, device=DEV))
            vp = guarded(torch.zeros((12, G, dv, PAGE), dtype=dtype, device=DEV))
            ops.qk_norm_temper_kv_write(qkv, t(np.ones(dk)), None, 1e-5, (0.5, 3), t(tok_pos, torch.int32), t(tok_seq, torch.int32),
                                        t(table, torch.int32), kp, vp, H, G, dk, dv, **prompt)
            pages.append((f64(qkv), f64(kp), f64(vp)))
        for a, b in zip(pages[0][:2], pages[1][:2]):          # q and k: the two kernels sum a head's squares in another order
            assert np.abs(a - b).max() <= (8e-3 if dtype == torch.bfloat16 else 1e-6) * np.abs(a).max()
        assert np.array_equal(pages[0][2], pages[1][2]) and np.abs(pages[0][2]).sum() > 0          # values are copies


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, dk, dv", [(3, 24, 40), (2, 128, 128), (1, 200, 16), (2, 64, 256), (1, 33, 4)])
def test_gla_step_of_one_token_a_sequence(ops, dtype, heads, dk, dv):
    """The fused step against the plain recurrence, norm and gate, from states that are not zero, on slots in
    another order than the sequences; and against the scan kernel with the separate norm and gate."""
    assert ops.gla_step_fits(dk, dv)
    rng = np.random.default_rng(dk + dv)
    B, tau = 3, 2.5
    proj = t(rng.normal(size=(B, 3 + 2 * heads * dk + 2 * heads * dv)), dtype)          # 3 unused | q | k | v | g
    q_off, k_off, v_off = 3, 3 + heads * dk, 3 + 2 * heads * dk
    g_off = v_off + heads * dv
    z, zb = rng.normal(size=(B, heads * dk)) * 3, rng.normal(size=heads * dk)
    slots = [5, 0, 3]
    state0 = rng.normal(size=(6, heads, dk, dv))
    gain = rng.normal(size=dv)
    state = t(state0)
    got = ops.gla_step(proj, q_off, k_off, v_off, g_off, t(z), t(zb), tau, dk ** -0.5, state, t(slots, torch.int32), t(gain),
                       1e-5, heads, dk, dv)
    p = f64(proj)
    alpha = Z.sigmoid(f64(t(z)) + f64(t(zb))) ** (1.0 / tau)
    want_state = state0.astype(np.float32).astype(np.float64)
    o = np.zeros((B, heads, dv))
    for b in range(B):
        for h in range(heads):
            o[b, h] = Z.gla_recurrence(p[b:b + 1, q_off + h * dk:q_off + (h + 1) * dk] * dk ** -0.5,
                                       p[b:b + 1, k_off + h * dk:k_off + (h + 1) * dk],
                                       p[b:b + 1, v_off + h * dv:v_off + (h + 1) * dv],
                                       alpha[b:b + 1, h * dk:(h + 1) * dk], want_state[slots[b], h])[0]
    want = Z.rms_norm(o, gain, 1e-5) * Z.silu(p[:, g_off:g_off + heads * dv].reshape(B, heads, dv))
    close(state, want_state, 5e-6, "state")
    close(got, want.reshape(B, -1), 1e-5 if dtype == torch.float32 else BF16_OUT, "step")
    assert ops.gla_step_fits(512, 512) is False and ops.gla_step_fits(64, 30) is False


def test_gla_token_by_token_is_the_scan(ops):
    """One call over 21 tokens against 21 calls of one token through the state, and against blocks of odd sizes."""
    rng = np.random.default_rng(2)
    heads, dk, dv, T = 2, 40, 24, 21
    proj = t(rng.normal(size=(T, 2 * heads * dk + heads * dv)))
    z, zb = t(rng.normal(size=(T, heads * dk)) * 2), t(rng.normal(size=heads * dk))
    offs = (0, heads * dk, 2 * heads * dk)

    def run(cuts):
        state = guarded(torch.zeros((2, heads, dk, dv), device=DEV))
        outs, at = [], 0
        for n in cuts:
            cu = t([0, n], torch.int32)
            outs.append(f64(ops.gla_scan(guarded(proj[at:at + n].clone()), *offs, guarded(z[at:at + n].clone()), zb, 2.0, 1.0,
                                         state, cu, t([1], torch.int32), heads, dk, dv)))
            at += n
        return np.concatenate(outs), f64(state)

    whole, s_whole = run([T])
    for cuts in ([1] * T, [2, 9, 1, 9], [8, 8, 5]):
        got, s = run(cuts)
        assert np.abs(got - whole).max() <= 1e-5 * np.abs(whole).max()
        assert np.abs(s - s_whole).max() <= 1e-5 * np.abs(s_whole).max()
    assert np.all(s_whole[0] == 0)                       # the other slot was not touched


@pytest.mark.parametrize("dtype, n", [(torch.float32, 1001), (torch.bfloat16, 4096), (torch.bfloat16, 77)])
def test_relu_squared(ops, dtype, n):
    y = t(np.random.default_rng(0).normal(size=n), dtype)
    close(ops.relu_squared(y), Z.relu_squared(f64(y)), F32 if dtype == torch.float32 else 4e-3)
