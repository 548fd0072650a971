"""One transformer layer of the reference's model graph (experiment/ModelIR/dolly-v2-3b-q0f16/before_dl.py, `prefill`
:2696-2746 and `decode` with n = 1), call by call through the library, against the same chain of oracle functions.

Two comparisons: every call's output against the oracle applied to that call's own (device) inputs, to the bar of the
op (bit-exact for the index-only ones), and the layer's output against the oracle chain run on its own from the layer's
inputs, where the fp16 roundings of a dozen calls accumulate."""
import numpy as np
import pytest
import torch

from dtas_amd import _lib, ops
from gpu_util import assert_bits_equal, dev

pytestmark = pytest.mark.gpu

H, HEADS, D, ROT, FF, VOCAB, MAX_POS = 2560, 32, 80, 20, 10240, 50280, 4096
RTOL = 1e-2          # GEMV / GEMM outputs
ATOL = 1e-2          # reductions


def _weights(seed=11):
    rng = np.random.default_rng(seed)
    f16 = lambda shape, std: (rng.standard_normal(shape) * std).astype(np.float16)
    f32 = lambda shape, lo, hi: rng.uniform(lo, hi, shape).astype(np.float32)
    pos = np.arange(MAX_POS)[:, None] / (10000.0 ** (np.arange(ROT)[None, :] % (ROT // 2) * 2.0 / ROT))
    return {
        "ln1_g": f32(H, 0.5, 1.5), "ln1_b": f32(H, -0.2, 0.2), "ln2_g": f32(H, 0.5, 1.5), "ln2_b": f32(H, -0.2, 0.2),
        "qkv_w": f16((3 * H, H), 0.02), "qkv_b": f16(3 * H, 0.02), "o_w": f16((H, H), 0.02), "o_b": f16(H, 0.02),
        "up_w": f16((FF, H), 0.02), "up_b": f16(FF, 0.02), "down_w": f16((H, FF), 0.01), "down_b": f16(H, 0.02),
        "cos": np.cos(pos).astype(np.float16), "sin": np.sin(pos).astype(np.float16),
    }


def _close(got, want, what, rtol=RTOL, atol=ATOL):
    g, w = got.astype(np.float64), want.astype(np.float64)
    bad = np.abs(g - w) > atol + rtol * np.abs(w)
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.size} outside tolerance, worst {np.abs(g - w).max():.4g}"


class Chain:
    """Runs one op on the device and checks it against the oracle on the same inputs."""

    def __init__(self, oracle):
        self.o = oracle

    def __call__(self, what, run, shape, dtype, ref, exact=False, **tol):
        out = torch.empty(shape, dtype=dtype, device="cuda")
        run(out)
        torch.cuda.synchronize()
        got, want = out.cpu().numpy(), ref()
        if exact:
            assert_bits_equal(got.reshape(want.shape), want)
        else:
            _close(got.reshape(want.shape), want, what, **tol)
        return out


def _layer_device(oracle, W, Wd, x, k_past, v_past):
    """x [n, H] fp16 (device), k_past / v_past [past, HEADS, D]: returns the layer's output and the new keys / values."""
    o, run = oracle, Chain(oracle)
    n, past = x.shape[0], k_past.shape[0]
    m = n + past
    host = lambda t: t.cpu().numpy()
    mask = run("mask", lambda out: ops.attn_mask(out), (1, 1, n, m), torch.float16, lambda: o.layout.attn_mask(n, m), exact=True)
    x32 = run("cast", lambda out: ops.cast(x, out), (n, H), torch.float32, lambda: o.c.cast(host(x), "float32"), exact=True)
    h1 = run("ln1", lambda out: ops.layer_norm(x32, Wd["ln1_g"], Wd["ln1_b"], out), (n, H), torch.float16,
             lambda: o.c.layer_norm(host(x32), W["ln1_g"], W["ln1_b"]), rtol=0)
    mm = ops.gemm if n > 1 else ops.gemv
    qkv = run("qkv", lambda out: mm(h1, Wd["qkv_w"], Wd["qkv_b"], out), (n, 3 * H), torch.float16,
              lambda: o.c.gemm(host(h1), W["qkv_w"], W["qkv_b"], threads=8))
    q = torch.empty(n, HEADS, D, dtype=torch.float16, device="cuda")
    k, v = torch.empty_like(q), torch.empty_like(q)
    ops.split3(qkv.view(n, HEADS, 3 * D), q, k, v)
    torch.cuda.synchronize()
    for got, want in zip((q, k, v), o.layout.split3(host(qkv).reshape(n, HEADS, 3 * D))):
        assert_bits_equal(host(got), want)
    rot = lambda a, name: run(name, lambda out: ops.rotary(a, Wd["cos"], Wd["sin"], out, m), (n, HEADS, D), torch.float16,
                              lambda: o.c.rotary(host(a), W["cos"], W["sin"], m), exact=True)
    q, k = rot(q, "rotary q"), rot(k, "rotary k")
    keys, values = torch.cat([k_past, k]), torch.cat([v_past, v])          # the cache append and view: the runtime's part
    swap = lambda a, name: run(name, lambda out: ops.swap_axes(a, out), (a.shape[1], a.shape[0], a.shape[2]), torch.float16,
                               lambda: o.layout.swap_axes(host(a)), exact=True)
    qh, kh, vh = swap(q, "transpose q"), swap(keys, "transpose k"), swap(values, "transpose v")
    scores = run("scores", lambda out: ops.attn_scores(qh, kh, mask, out), (HEADS, n, m), torch.float32,
                 lambda: o.c.attn_scores(host(qh), host(kh), host(mask).reshape(n, m), 0.11179039301310044, threads=8))
    probs = run("softmax", lambda out: ops.softmax(scores, out), (HEADS, n, m), torch.float16,
                lambda: o.c.softmax(host(scores), threads=8), rtol=0)
    ctx = run("pv", lambda out: ops.attn_pv(probs, vh, out), (HEADS, n, D), torch.float16,
              lambda: o.c.attn_pv(host(probs), host(vh), threads=8))
    merged = swap(ctx, "transpose out").view(n, H)
    h2 = run("ln2", lambda out: ops.layer_norm(x32, Wd["ln2_g"], Wd["ln2_b"], out), (n, H), torch.float16,
             lambda: o.c.layer_norm(host(x32), W["ln2_g"], W["ln2_b"]), rtol=0)
    up = run("up+gelu", lambda out: mm(h2, Wd["up_w"], Wd["up_b"], out, epilogue=_lib.EPI_BIAS_GELU), (n, FF), torch.float16,
             lambda: o.c.gemm_fused(host(h2), W["up_w"], W["up_b"], None, None, 3, threads=8))
    down = run("down", lambda out: mm(up, Wd["down_w"], Wd["down_b"], out), (n, H), torch.float16,
               lambda: o.c.gemm(host(up), W["down_w"], W["down_b"], threads=8))
    y = run("out+add+add", lambda out: mm(merged, Wd["o_w"], Wd["o_b"], out, epilogue=_lib.EPI_BIAS_ADD2, res1=down, res2=x),
            (n, H), torch.float16, lambda: o.c.gemm_fused(host(merged), W["o_w"], W["o_b"], host(down), host(x), 1, threads=8))
    return y, keys, values


def _layer_oracle(o, W, x, k_past, v_past):
    n, m = x.shape[0], x.shape[0] + k_past.shape[0]
    x32 = o.c.cast(x, "float32")
    qkv = o.c.gemm(o.c.layer_norm(x32, W["ln1_g"], W["ln1_b"]), W["qkv_w"], W["qkv_b"], threads=8)
    q, k, v = o.layout.split3(qkv.reshape(n, HEADS, 3 * D))
    q, k = o.c.rotary(q, W["cos"], W["sin"], m), o.c.rotary(k, W["cos"], W["sin"], m)
    keys, values = np.concatenate([k_past, k]), np.concatenate([v_past, v])
    scores = o.c.attn_scores(o.layout.swap_axes(q), o.layout.swap_axes(keys), o.layout.attn_mask(n, m), 0.11179039301310044, threads=8)
    ctx = o.c.attn_pv(o.c.softmax(scores, threads=8), o.layout.swap_axes(values), threads=8)
    merged = o.layout.swap_axes(ctx).reshape(n, H)
    up = o.c.gemm_fused(o.c.layer_norm(x32, W["ln2_g"], W["ln2_b"]), W["up_w"], W["up_b"], None, None, 3, threads=8)
    down = o.c.gemm(up, W["down_w"], W["down_b"], threads=8)
    return o.c.gemm_fused(merged, W["o_w"], W["o_b"], down, x, 1, threads=8), keys, values


@pytest.mark.parametrize("n,past", [(37, 0), (64, 0), (19, 45), (1, 63), (1, 0)])
def test_one_layer_call_by_call(oracle, n, past):
    W = _weights()
    Wd = {k: dev(v) for k, v in W.items()}
    rng = np.random.default_rng(n * 100 + past)
    x = rng.standard_normal((n, H)).astype(np.float16)
    k_past = (rng.standard_normal((past, HEADS, D)) * 0.5).astype(np.float16)
    v_past = (rng.standard_normal((past, HEADS, D)) * 0.5).astype(np.float16)
    y, keys, values = _layer_device(oracle, W, Wd, dev(x), dev(k_past), dev(v_past))
    want, wkeys, wvalues = _layer_oracle(oracle, W, x, k_past, v_past)
    # the chains run apart from the layer's inputs on: a last-place difference in one call moves the next call's input
    _close(keys.cpu().numpy(), wkeys, "keys", rtol=2e-2, atol=2e-2)
    _close(values.cpu().numpy(), wvalues, "values", rtol=2e-2, atol=2e-2)
    got = y.cpu().numpy().astype(np.float64)
    assert np.abs(got - want.astype(np.float64)).max() < 5e-2 and np.abs(got - want.astype(np.float64)).mean() < 2e-3


def test_sampling_head(oracle):
    """layer_norm (the last one, fp32), slice + fused_slice1_cast4 (the last position), NT_matmul5 (the vocabulary
    projection) and softmax_with_temperature (before_dl.py:4144, :2677-2679, :4154-4161)."""
    rng = np.random.default_rng(5)
    n = 9
    hidden = rng.standard_normal((n, H)).astype(np.float32)
    g, b = rng.uniform(0.5, 1.5, H).astype(np.float32), rng.uniform(-0.2, 0.2, H).astype(np.float32)
    emb = (rng.standard_normal((VOCAB, H)) * 0.05).astype(np.float32)
    normed = torch.empty(n, H, dtype=torch.float32, device="cuda")
    ops.layer_norm_f32(dev(hidden), dev(g), dev(b), normed)
    last = torch.empty(1, H, dtype=torch.float32, device="cuda")
    ops.copy(normed[n - 1:], last)
    logits = torch.empty(1, VOCAB, dtype=torch.float32, device="cuda")
    ops.gemv_f32(last, dev(emb), logits)
    probs = torch.empty_like(logits)
    ops.softmax_temperature(logits, torch.tensor(0.7, dtype=torch.float32, device="cuda"), probs)
    torch.cuda.synchronize()
    want_normed = oracle.c.layer_norm_f32(hidden, g, b)
    assert np.abs(normed.cpu().numpy() - want_normed).max() < 1e-4
    assert torch.equal(last[0], normed[n - 1])
    want_logits = oracle.c.gemv_f32(want_normed[n - 1], emb, threads=8).reshape(1, VOCAB)
    _close(logits.cpu().numpy(), want_logits, "logits", atol=1e-3)
    want = oracle.c.softmax_temperature(want_logits, 0.7)
    got = probs.cpu().numpy()
    assert np.abs(got - want).max() < 1e-2 and np.abs(got / want - 1).max() < 2e-2
    assert int(got.argmax()) == int(want.argmax()) and abs(float(got.astype(np.float64).sum()) - 1) < 1e-4


def _decode_step(Ws, caches, bufs, x, cos, sin, m):
    """The decode graph's layers (n = 1) as plain launches on the current stream: no checks, no synchronisation, every
    buffer allocated beforehand -- what a caller records into a HIP graph."""
    n, cur = 1, x
    for W, (kh, vh), b in zip(Ws, caches, bufs):
        ops.attn_mask(b["mask"])
        ops.cast(cur, b["x32"])
        ops.layer_norm(b["x32"], W["ln1_g"], W["ln1_b"], b["h1"])
        ops.gemv(b["h1"], W["qkv_w"], W["qkv_b"], b["qkv"])
        ops.split3(b["qkv"].view(n, HEADS, 3 * D), b["q"], b["k"], b["v"])
        ops.rotary(b["q"], cos, sin, b["qr"], m)
        ops.rotary(b["k"], cos, sin, b["kr"], m)
        kh[:, m - 1, :].copy_(b["kr"][0])                         # the cache append: the runtime's part
        vh[:, m - 1, :].copy_(b["v"][0])
        ops.swap_axes(b["qr"], b["qh"])
        ops.attn_scores(b["qh"], kh, b["mask"], b["scores"])
        ops.softmax(b["scores"], b["probs"])
        ops.attn_pv(b["probs"], vh, b["ctx"])
        ops.swap_axes(b["ctx"], b["merged"])
        ops.layer_norm(b["x32"], W["ln2_g"], W["ln2_b"], b["h2"])
        ops.gemv(b["h2"], W["up_w"], W["up_b"], b["up"], epilogue=_lib.EPI_BIAS_GELU)
        ops.gemv(b["up"], W["down_w"], W["down_b"], b["down"])
        ops.gemv(b["merged"].view(n, H), W["o_w"], W["o_b"], b["y"], epilogue=_lib.EPI_BIAS_ADD2, res1=b["down"], res2=cur)
        cur = b["y"]
    return cur


@pytest.mark.parametrize("past", [63, 4000])      # (4000 keys: P.V shares the keys between workgroups through the workspace)
def test_decode_layers_recorded_into_a_graph_replay_the_same_bits(past):
    """Two layers of the decode step recorded into a HIP graph (the launch-bound loop of serving: 20 launches of a few
    microseconds per layer) and replayed three times, with eager launches on the same stream's workspace between the
    replays; every replay gives the bits of the eager run.  The stream is warmed up first: a workspace is allocated at
    a stream's first split launch, and nothing may allocate while a graph is recorded."""
    W = _weights()
    layers, m = 2, past + 1
    Wd = {k: dev(v) for k, v in W.items()}
    rng = np.random.default_rng(past)
    x = dev(rng.standard_normal((1, H)).astype(np.float16))
    cache = lambda: dev((rng.standard_normal((HEADS, m, D)) * 0.5).astype(np.float16))
    caches = [(cache(), cache()) for _ in range(layers)]
    E = lambda *s, dt=torch.float16: torch.empty(*s, dtype=dt, device="cuda")
    bufs = [dict(mask=E(1, 1, 1, m), x32=E(1, H, dt=torch.float32), h1=E(1, H), qkv=E(1, 3 * H), q=E(1, HEADS, D), k=E(1, HEADS, D),
                 v=E(1, HEADS, D), qr=E(1, HEADS, D), kr=E(1, HEADS, D), qh=E(HEADS, 1, D), scores=E(HEADS, 1, m, dt=torch.float32),
                 probs=E(HEADS, 1, m), ctx=E(HEADS, 1, D), merged=E(1, HEADS, D), h2=E(1, H), up=E(1, FF), down=E(1, H), y=E(1, H))
            for _ in range(layers)]
    step = lambda: _decode_step([Wd] * layers, caches, bufs, x, Wd["cos"], Wd["sin"], m)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        eager = step().clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        y = step()
    a, w, c = torch.randn(40, 2048, device="cuda").half(), torch.randn(1000, 2048, device="cuda").half(), E(40, 1000)
    for _ in range(3):
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert_bits_equal(y.cpu().numpy(), eager.cpu().numpy())
        with torch.cuda.stream(side):       # eager work between the replays: a split GEMM and another sequence length's P.V
            ops.gemm(a, w, None, c)
            ops.attn_pv(torch.rand(HEADS, 1, 3500, device="cuda").half(), torch.randn(HEADS, 3500, D, device="cuda").half(), E(HEADS, 1, D))
        torch.cuda.synchronize()
