"""Vobisun (parallel layers; windowed attention with pooled blocks and a sink beside gated linear attention; looped layers) on the GPU against
the plain float64 statement in tests/seq_oracle.py: small configurations and weights made here, every schedule (whole prompts, token by
token, portions down to two tokens, interleaved requests, reused slots, ring wrap, long decoding, greedy generation), and a hand-made model
in which ONE key carries most of the weight, so that a window one token off, a block seen too early or too late or a lost far key shows."""
import numpy as np
import pytest

import seq_oracle
from powerserve_amd import hip, host, seqmodel, synth
from powerserve_amd.safetensors_io import f32_to_bf16_bits

pytestmark = pytest.mark.gpu

PL, PC = synth.parallel_layer, synth.parallel_config


def att(heads, kv_heads, dim, vdim, size, pool, dims, base=100.0, factor=None, scale=0.3):
    rot = {"base": base, "dims": dims}
    if factor:
        rot["scaling"] = {"factor": factor}
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, mask={"size": size, "pool": pool}, rot=rot, scale=scale)


def gla(heads, dim, vdim, tau):
    return dict(heads=heads, dim=dim, vdim=vdim, tau=tau)


CONFIGS = {
    # sizes that are multiples of nothing (per-key attention kernel), kv_heads == heads, the whole head rotated, no position scaling, one tap,
    # a window of one with blocks of one, a layer without feed-forward, no loop
    "odd": PC(40, 50, [PL(28, att(3, 3, 10, 6, 5, 2, 10), gla(2, 7, 9, 2.0), 1.3, 0.6),
                       PL(None, att(4, 1, 6, 10, 1, 1, 2, base=7.0, factor=3.0), gla(1, 20, 5, 16.0), 0.8, 1.1)], taps=1, eps=1e-5, embed_scale=2.0),
    # sizes the matrix-core kernels take; a looped stretch (five layer runs over three layers)
    "aligned": PC(128, 96, [PL(192, att(4, 2, 32, 16, 33, 5, 16, base=500.0, factor=4.0, scale=0.2), gla(2, 64, 32, 8.0), 1.2, 1.1),
                            PL(64, att(2, 2, 16, 64, 9, 4, 8), gla(4, 16, 16, 1.0), 1.0, 1.0),
                            PL(None, att(4, 1, 16, 32, 20, 20, 16, scale=0.25), gla(1, 32, 64, 4.0), 0.5, 1.5)], taps=3, embed_scale=4.0, loop=(1, 3, 2)),
    # more heads in a key / value group than a tile of the single-token kernel has rows; the loop covers everything, three times
    "manyheads": PC(64, 40, [PL(48, att(20, 1, 16, 8, 40, 16, 4), gla(1, 8, 8, 2.0))], taps=2, loop=(0, 1, 3)),
    # recurrent heads of more than 64 rows (state rows over 16 lanes), 128 value columns per attention head
    "wide": PC(96, 40, [PL(None, att(2, 2, 48, 128, 12, 4, 32), gla(2, 144, 72, 16.0))], taps=4),
}
TOL = {"float32": 2e-4, "bfloat16": 1e-1}  # fp32: a few ulps of fp32 sums; bfloat16: 8-bit mantissas in models this narrow


def err(got, want):
    """centred rms of the difference over the rms of the logits, worst row"""
    d = np.asarray(got, dtype=np.float64) - want
    d = d - d.mean(-1, keepdims=True)
    s = np.sqrt(np.mean((want - want.mean(-1, keepdims=True)) ** 2))
    return float(np.sqrt(np.mean(d * d, -1)).max() / s)


def rows(got, want, which):
    return [err(got[i:i + 1], want[i:i + 1]) for i in which]


@pytest.fixture(scope="module")
def made(ctx, tmp_path_factory):
    cache = {}

    def get(name, dtype="float32", max_batch=16, cfg=None, tensors=None, max_context=1024):
        key = (name, dtype, max_batch, max_context)
        if key not in cache:
            c = cfg or CONFIGS[name]
            d = str(tmp_path_factory.mktemp("p"))
            t = synth.write_seq_model_dir(d, c, 0, tensors)
            cache[key] = (seqmodel.load_model(ctx, d, dtype=dtype, max_batch=max_batch, n_slots=3, max_context=max_context), c, t)
        return cache[key]

    yield get
    for m, _, _ in cache.values():
        m.close()


def tokens_for(cfg, n, seed=1, lo=0):
    return np.random.default_rng(seed).integers(lo, cfg["vocab"], n).astype(np.int32)


def run_portions(m, toks, sizes):
    s, out, at, i = m.acquire(), [], 0, 0
    while at < len(toks):
        n = min(sizes[i % len(sizes)], len(toks) - at)
        out.append(m.forward(s, toks[at:at + n], np.arange(n)))
        at, i = at + n, i + 1
    m.release(s)
    return np.concatenate(out)


def bf16(t):
    return {k: (f32_to_bf16_bits(np.asarray(v, np.float32)).astype(np.uint32) << 16).view(np.float32).reshape(np.shape(v)) for k, v in t.items()}


# ---------------------------------------------------------------------------------------------------------------- mechanisms, one at a time
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["attention", "attention_mfma", "linear", "feed_forward"])
def test_each_mechanism_alone(made, which, dtype):
    """one layer in which only one of the three sublayers contributes: what it adds to the residual stream against that mechanism's own plain function"""
    a = att(4, 2, 16, 8, 6, 3, 8, factor=2.0) if which == "attention_mfma" else att(3, 1, 10, 6, 6, 3, 6, factor=2.0)
    g = gla(2, 12, 20, 3.0)
    ls, rs, ff = {"attention": (1.4, 0.0, None), "attention_mfma": (0.9, 0.0, None), "linear": (0.0, 0.7, None), "feed_forward": (0.0, 0.0, 36)}[which]
    cfg = PC(40, 32, [PL(ff, a, g, ls, rs)], taps=3, eps=1e-5, embed_scale=1.5)
    m, _, t = made("alone_" + which, dtype, max_batch=32, cfg=cfg)
    toks = tokens_for(cfg, 30, seed=3)
    W = {k: np.asarray(v, np.float64) for k, v in t.items()}
    x0 = W["embed"][toks] * 1.5
    h = seq_oracle.plain_norm(x0, W["l0.norm1"], 1e-5)
    hm = h + seq_oracle.time_conv(h, W["l0.canon1"])
    want = {"attention": lambda: ls * seq_oracle.pooled_window_attention(W, "l0.mix.left.", hm, a, 1e-5),
            "attention_mfma": lambda: ls * seq_oracle.pooled_window_attention(W, "l0.mix.left.", hm, a, 1e-5),
            "linear": lambda: rs * seq_oracle.gated_linear_attention(W, "l0.mix.right.", hm, g, 1e-5),
            "feed_forward": lambda: seq_oracle.gated_feed_forward(W, "l0.mlp.", h)}[which]()
    m.capture_layers(True)
    s = m.acquire()
    m.forward(s, toks)
    got = m.layers(len(toks))[0].astype(np.float64) - x0
    m.release(s)
    m.capture_layers(False)
    assert np.abs(got - want).max() < (2e-4 if dtype == "float32" else 6e-2) * np.abs(want).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "aligned", "manyheads", "wide"])
def test_whole_prompt_against_the_plain_statement(made, name, dtype):
    m, cfg, t = made(name, dtype, max_batch=64)
    toks = tokens_for(cfg, 70)
    want = seq_oracle.run_parallel(cfg, t, toks)
    s = m.acquire()
    got = m.forward(s, toks, np.arange(len(toks)))
    m.release(s)
    assert err(got, want) < TOL[dtype]


@pytest.mark.parametrize("name", ["odd", "aligned", "manyheads"])
def test_residual_stream_after_every_layer_run(made, name):
    m, cfg, t = made(name, "float32", max_batch=64)
    toks = tokens_for(cfg, 45, seed=5)
    per = []
    seq_oracle.run_parallel(cfg, t, toks, per_layer=per)
    assert m.n_runs == len(per) == len(seq_oracle.layer_runs(cfg))
    m.capture_layers(True)
    s = m.acquire()
    m.forward(s, toks)
    got = m.layers(len(toks))
    m.release(s)
    m.capture_layers(False)
    for i, want in enumerate(per):
        assert np.abs(got[i] - want).max() < 2e-4 * np.abs(want).max(), i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["odd", "aligned", "manyheads", "wide"])
def test_token_by_token_and_portions_give_the_whole_prompts_logits(made, name, dtype):
    m, cfg, t = made(name, dtype, max_batch=16)  # 16: a 50-token portion is also cut inside the library
    toks = tokens_for(cfg, 90, seed=2)
    want = seq_oracle.run_parallel(cfg, t, toks)
    for sizes in ([1], [2], [3, 1, 7, 2], [50, 2, 23], [16, 17, 15]):
        assert err(run_portions(m, toks, sizes), want) < TOL[dtype], sizes


def test_first_tokens_of_a_sequence(made):
    m, cfg, t = made("aligned", "float32")
    for n in (1, 2, 3, 5):
        toks = tokens_for(cfg, n, seed=10 + n)
        want = seq_oracle.run_parallel(cfg, t, toks)
        assert err(run_portions(m, toks, [n]), want) < TOL["float32"]
        assert err(run_portions(m, toks, [1]), want) < TOL["float32"]


def test_interleaved_requests_and_reused_slots(made):
    """requests of unequal length fed in turns through the scheduler against each alone; then every slot is used again and must start from nothing"""
    m, cfg, t = made("aligned", "float32", max_batch=16)
    seqs = [tokens_for(cfg, n, seed=20 + n) for n in (61, 9, 88)]
    want = [seq_oracle.run_parallel(cfg, t, s) for s in seqs]
    sched = seqmodel.RequestScheduler(m)
    got, at = [[] for _ in seqs], [0, 0, 0]
    steps, i = [5, 2, 11, 1, 3], 0
    while any(a < len(s) for a, s in zip(at, seqs)):
        r = i % 3
        if at[r] < len(seqs[r]):
            n = min(steps[i % len(steps)], len(seqs[r]) - at[r])
            got[r].append(sched.feed("req%d" % r, seqs[r][at[r]:at[r] + n], np.arange(n)))
            at[r] += n
            if at[r] == len(seqs[r]):
                sched.finish("req%d" % r)
        i += 1
    for g, w in zip(got, want):
        assert err(np.concatenate(g), w) < TOL["float32"]
    for r in range(4):
        assert err(sched.feed("again", seqs[2], np.arange(len(seqs[2]))), want[2]) < TOL["float32"]
        sched.finish("again")
    with pytest.raises(hip.PSHipError):
        [m.acquire() for _ in range(4)]
    for s in range(3):
        m.release(s)


# ---------------------------------------------------------------------------------------------------------------- one key that stands out
def marked_model(size, pool, aligned, seed=0):
    """Token 0 is a MARK: its embedding alone has feature 0; every key reads feature 0 into one unrotated channel of its head and every query has a
    constant in that channel (a bias), so a query's score for a mark it can see is far above all others, directly and (divided by the block size) through
    its block's mean; every value channel reads feature 0 too, so the mark's value is a constant the other tokens do not have.  Whether a query sees
    the mark -- in its window, through a block, or not at all -- decides its logits."""
    rng = np.random.default_rng(seed)
    W, V = 32, 24
    H, G, d, dv = (4, 2, 16, 8) if aligned else (3, 1, 10, 6)
    a = att(H, G, d, dv, size, pool, 4, base=50.0, factor=2.0, scale=1.0)
    cfg = PC(W, V, [PL(None, a, gla(1, 8, 8, 4.0), 1.0, 0.3), PL(24, att(2, 2, 8, 8, 5, 2, 8), gla(2, 8, 8, 2.0))], taps=2, eps=1e-5, embed_scale=1.0)
    t = synth.seq_tensors(cfg, seed)
    e = rng.standard_normal((V, W)).astype(np.float32)
    e[:, 0] = 0.0
    e[0, 0] = 6.0
    t["embed"] = e
    t["l0.norm1"], t["l0.canon1"] = np.ones(W, np.float32), np.zeros((W, 2), np.float32)
    c = d - 1                                    # a channel the rotation leaves alone (4 of a head's numbers turn)
    k = rng.standard_normal((G * d, W)).astype(np.float32) * 0.1
    k[:, 0] = 0.0
    q = rng.standard_normal((H * d, W)).astype(np.float32) * 0.1
    qb, kb = np.zeros(H * d, np.float32), np.zeros(G * d, np.float32)
    for g in range(G):
        k[g * d + c, 0] = 3.0
    for h in range(H):
        qb[h * d + c] = 2.0
    v = rng.standard_normal((G * dv, W)).astype(np.float32) * 0.2
    v[:, 0] = 1.5                                # the mark's value: a constant the other tokens do not have
    p = "l0.mix.left."
    t[p + "q"], t[p + "q.b"], t[p + "k"], t[p + "k.b"], t[p + "v"], t[p + "v.b"] = q, qb, k, kb, v, np.zeros(G * dv, np.float32)
    t[p + "q.norm"], t[p + "k.norm"] = np.ones(H * d, np.float32), np.ones(G * d, np.float32)
    t[p + "temp"], t[p + "sink"] = np.full(H, 1.5, np.float32), np.full(H, 2.0, np.float32)
    return cfg, bf16(t)


def marked_tokens(cfg, n, marks, seed):
    toks = tokens_for(cfg, n, seed, lo=1)
    toks[list(marks)] = 0
    return toks


@pytest.mark.parametrize("aligned", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_and_block_edges_in_prompts_and_in_decoding(made, dtype, aligned):
    """Marks at 3 and 30, window 11, blocks of 4.  The mark at 30 is in the window up to position 40, unseen at 41 .. 42 (its block 28 .. 31 is seen from
    31 + 11 = 42 on).  The plain statement with the window one longer or shorter, with blocks of another size or without the sink is far off on exactly
    those rows; the library agrees with the right one however the tokens are cut: edges inside a prompt, at portion borders, on decoded tokens."""
    size, pool = 11, 4
    cfg, t = marked_model(size, pool, aligned)
    m, _, _ = made("marked%d" % aligned, dtype, max_batch=8, cfg=cfg, tensors=t)
    toks = marked_tokens(cfg, 80, (3, 30), seed=3)
    want = seq_oracle.run_parallel(cfg, t, toks)
    wrong = lambda **kw: seq_oracle.run_parallel(cfg, t, toks, **kw)
    assert min(rows(wrong(size=size + 1), want, [41])) > 0.2 and min(rows(wrong(size=size - 1), want, [40])) > 0.2
    assert min(rows(wrong(pool=pool + 1), want, [42, 43])) > 0.05 and min(rows(wrong(pool=2), want, [41])) > 0.05
    assert min(rows(wrong(use_sink=False), want, [0, 1, 2])) > 0.02
    tol = 1e-3 if dtype == "float32" else TOL[dtype]
    for sizes in ([80], [1], [2], [8], [5, 2, 12, 1], [40, 1, 1, 1, 1], [41, 1, 1, 1], [42, 2, 1], [31, 10, 1, 1, 1]):
        got = run_portions(m, toks, sizes)
        assert max(rows(got, want, range(len(toks)))) < tol, sizes


@pytest.mark.parametrize("aligned", [False, True])
def test_far_key_among_hundreds_and_a_ring_that_wraps(made, aligned):
    """window 200, blocks of 7: the mark 199 tokens back still carries the weight, one token later it is gone until its block is seen.  A 230-token
    prompt in portions of 64, then 200 single tokens: the ring (263 rows) wraps, and the far key is first a prompt token (mark at 10: last seen in the
    window at 209), then a decoded one (mark at 215: at 414); no second mark is in sight at either edge."""
    size, pool = 200, 7
    cfg, t = marked_model(size, pool, aligned, seed=1)
    m, _, _ = made("far%d" % aligned, "float32", max_batch=64, cfg=cfg, tensors=t)
    toks = marked_tokens(cfg, 430, (10, 215), seed=4)
    want = seq_oracle.run_parallel(cfg, t, toks)
    assert min(rows(seq_oracle.run_parallel(cfg, t, toks, size=size - 1), want, [209, 414])) > 0.2
    assert min(rows(seq_oracle.run_parallel(cfg, t, toks, size=size + 1), want, [210, 415])) > 0.2
    s = m.acquire()
    got = [m.forward(s, toks[:230], np.arange(230))] + [m.forward(s, toks[i:i + 1], [0]) for i in range(230, 430)]
    m.release(s)
    assert max(rows(np.concatenate(got), want, range(len(toks)))) < 1e-3


def test_long_decoding_keeps_the_states(made):
    m, cfg, t = made("aligned", "float32", max_batch=16)
    toks = tokens_for(cfg, 260, seed=6)
    want = seq_oracle.run_parallel(cfg, t, toks)
    assert err(run_portions(m, toks, [13, 1, 1, 1, 1, 1, 1, 1]), want) < TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["aligned", "odd"])
def test_greedy_generation_through_the_entry_point(made, name, dtype):
    """SeqModel.generate (prefill, then the captured single-token step feeding its own arg-max) picks, at every step, a token whose logit in the
    plain statement is the largest up to rounding; eager launches and a host sampler set to top-1 give the same ids."""
    m, cfg, t = made(name, dtype, max_batch=16)
    prompt = tokens_for(cfg, 29, seed=7)
    ids = m.generate(prompt, 40)
    assert ids.shape == (40,)
    full = np.concatenate([prompt, ids])
    want = seq_oracle.run_parallel(cfg, t, full[:-1])
    spread = want.max() - want.min()
    for i, tok in enumerate(ids):
        row = want[len(prompt) - 1 + i]
        assert row.max() - row[tok] < (1e-4 if dtype == "float32" else 3e-2) * spread, i
    m.set_mode(1)
    assert np.array_equal(m.generate(prompt, 40), ids)
    m.set_mode(0)
    assert np.array_equal(m.generate(prompt, 40), ids)  # the captured sequence replayed on a slot that was used before
    sm = host.Sampler(host.SamplerCfg.make(cfg["vocab"], seed=1, temperature=1.0, top_p=1.0, top_k=1))
    assert np.array_equal(m.generate(prompt, 40, sampler=sm.sample), ids)
    sm.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["aligned", "manyheads", "wide"])
def test_matrix_core_forms_agree_with_the_plain_kernels(made, name, dtype):
    """mode bit 1 keeps the per-key attention and the 64 x 64 mat-mul: the wide mat-mul, the mat-vec with its paired epilogue and the matrix-core
    attention of a portion and of a single token must give the same logits (fp32: up to the order of sums)"""
    m, cfg, t = made(name, dtype, max_batch=64)
    toks = tokens_for(cfg, 150, seed=9)
    fast = [run_portions(m, toks, sizes) for sizes in ([64], [1], [40, 1, 1, 1, 9])]
    m.set_mode(2)
    plain = [run_portions(m, toks, sizes) for sizes in ([64], [1], [40, 1, 1, 1, 9])]
    m.set_mode(0)
    want = seq_oracle.run_parallel(cfg, t, toks)
    for a, b in zip(fast, plain):
        assert err(a, b) < (1e-4 if dtype == "float32" else TOL[dtype])
        assert err(a, want) < TOL[dtype]


def test_host_facade_loads_and_generates_the_same(made, tmp_path):
    m, cfg, t = made("aligned", "float32", max_batch=16)
    synth.write_seq_model_dir(str(tmp_path), cfg, 0, t)
    hm = host.HostSeqModel(str(tmp_path), dtype="float32", max_batch=16, n_slots=2)
    prompt = tokens_for(cfg, 19, seed=7)
    ids = m.generate(prompt, 12)
    assert np.array_equal(hm.generate(prompt, 12), ids)
    s, s2 = hm.acquire(), m.acquire()
    a, b = hm.forward(s, prompt, [0, 5, 18]), m.forward(s2, prompt, [0, 5, 18])
    hm.release(s)
    m.release(s2)
    assert np.array_equal(a, b)
    hm.close()


def test_a_sequence_longer_than_the_context_is_refused(ctx, tmp_path):
    cfg = CONFIGS["odd"]
    synth.write_seq_model_dir(str(tmp_path), cfg, 0)
    m = seqmodel.load_model(ctx, str(tmp_path), dtype="float32", max_batch=8, n_slots=1, max_context=20)
    s = m.acquire()
    m.forward(s, tokens_for(cfg, 18))
    with pytest.raises(hip.PSHipError):
        m.forward(s, [1, 2, 3])
    m.forward(s, [1, 2])
    m.release(s)
    m.close()
