"""Layer-list models on the GPU against the plain float64 statement in tests/seq_oracle.py: small configurations and random weights made
here, every schedule (whole prompts, token by token, portions, interleaved requests, reused slots, ring wrap, greedy generation)."""
import numpy as np
import pytest

import seq_oracle
from powerserve_amd import hip, host, seqmodel, synth
from powerserve_amd.safetensors_io import f32_to_bf16_bits

pytestmark = pytest.mark.gpu

L = synth.seq_layer
LAT = dict(rot={"base": 10000.0, "dims": 8}, rot_dim=8)
CONFIGS = {
    # sizes that are multiples of nothing in particular; unequal taps; a layer without feed-forward
    "mixed": synth.seq_config(48, 64, [L("wkv", 40, heads=2, dim=24), L("delta", None, heads=4, kv_heads=2, dim=12, vdim=20, conv=4),
                                       L("latent_attention", 56, heads=3, dim=16, vdim=24, q_rank=20, kv_rank=28, mask={"size": 9}, scale=0.3, **LAT)],
                              taps=2, logit_scale=0.5),
    # sizes on the matrix cores' grid, other order of layers
    "aligned": synth.seq_config(128, 96, [L("latent_attention", 192, heads=2, dim=32, vdim=64, q_rank=48, kv_rank=64, mask={"size": 33}, scale=0.125,
                                            rot={"base": 500.0, "dims": 16}, rot_dim=16),
                                          L("delta", 128, heads=2, kv_heads=2, dim=64, vdim=32, conv=3), L("wkv", 128, heads=2, dim=64)], taps=3, eps=1e-5),
    # heads of more than 64 rows (state rows spread over 8 and 16 lanes), one head, one tap (no tail at all), window of one
    "wide_heads": synth.seq_config(80, 50, [L("wkv", 32, heads=1, dim=80), L("delta", 32, heads=3, kv_heads=1, dim=144, vdim=72, conv=1),
                                            L("latent_attention", None, heads=1, dim=8, vdim=70, q_rank=9, kv_rank=11, mask={"size": 1}, scale=1.0,
                                              rot={"base": 100.0, "dims": 2}, rot_dim=6)], taps=1),
    "wkv": synth.seq_config(40, 32, [L("wkv", None, heads=2, dim=20)], taps=4),
    "delta": synth.seq_config(40, 32, [L("delta", None, heads=2, kv_heads=1, dim=20, vdim=12, conv=2)], taps=3),
    "latent": synth.seq_config(40, 32, [L("latent_attention", None, heads=2, dim=12, vdim=20, q_rank=16, kv_rank=24, mask={"size": 6}, scale=0.4, **LAT)], taps=3),
    "ff": synth.seq_config(40, 32, [L("wkv", 24, heads=1, dim=8)], taps=2),
}
# float32: a few ulps of fp32 sums.  bfloat16: the operands of every matrix product are rounded to 8 bits of mantissa, which in models this
# narrow (48 to 128 channels) leaves 1-3 % on a typical row and up to 7 % on the worst of a hundred rows, whatever the schedule
TOL = {"float32": 2e-4, "bfloat16": 1e-1}


def err(got, want):
    """centred rms of the difference over the rms of the logits, worst row"""
    d = np.asarray(got, dtype=np.float64) - want
    d = d - d.mean(-1, keepdims=True)
    s = np.sqrt(np.mean((want - want.mean(-1, keepdims=True)) ** 2))
    return float(np.sqrt(np.mean(d * d, -1)).max() / s)


@pytest.fixture(scope="module")
def made(ctx, tmp_path_factory):
    """(name, dtype, max_batch) -> (model, cfg, tensors); models are built once and closed at the end"""
    cache = {}

    def get(name, dtype="float32", max_batch=16, seed=0, cfg=None, tensors=None):
        key = (name, dtype, max_batch, seed)
        if key not in cache:
            c = cfg or CONFIGS[name]
            d = str(tmp_path_factory.mktemp("m"))
            t = synth.write_seq_model_dir(d, c, seed, tensors)
            cache[key] = (seqmodel.load_model(ctx, d, dtype=dtype, max_batch=max_batch, n_slots=3), c, t)
        return cache[key]

    yield get
    for m, _, _ in cache.values():
        m.close()


def tokens_for(cfg, n, seed=1):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], n).astype(np.int32)


def run_portions(m, toks, sizes):
    """the sequence cut into portions of the given sizes (cycled), all logits"""
    s, out, at, i = m.acquire(), [], 0, 0
    while at < len(toks):
        n = min(sizes[i % len(sizes)], len(toks) - at)
        out.append(m.forward(s, toks[at:at + n], np.arange(n)))
        at, i = at + n, i + 1
    m.release(s)
    return np.concatenate(out)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,N,K", [(1, 37, 50), (2, 64, 96), (3, 19, 7), (8, 130, 72), (9, 70, 33), (70, 129, 200), (200, 48, 48), (1, 16, 4096)])
def test_dense_matmul_any_shape(ctx, dtype, T, N, K):
    rng = np.random.default_rng(T * 1000 + N)
    w = rng.standard_normal((N, K), dtype=np.float32)
    x = rng.standard_normal((T, K), dtype=np.float32)
    from powerserve_amd.safetensors_io import f32_to_bf16_bits
    bits = f32_to_bf16_bits(w)
    rnd = lambda a: (f32_to_bf16_bits(a).astype(np.uint32) << 16).view(np.float32).reshape(a.shape)
    import ctypes as C
    h = C.c_void_p()
    ctx.check(ctx.L.ps_hip_dense_upload(ctx.h, bits.ctypes.data_as(C.c_void_p), N, K, int(dtype == "float32"), C.byref(h)))
    dx, do = ctx.to_device(x), ctx.empty((T, N))
    ctx.check(ctx.L.ps_hip_dense_matmul(ctx.h, h, dx.ptr, T, do.ptr, 0.5))
    ctx.sync()
    xr = x if dtype == "float32" else rnd(x)
    want = 0.5 * (xr.astype(np.float64) @ rnd(w).astype(np.float64).T)
    assert np.abs(do.numpy() - want).max() < 1e-4 * max(1.0, np.abs(want).max())
    ctx.L.ps_hip_dense_free(ctx.h, h)
    dx.free(); do.free()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["wkv", "delta", "latent", "ff", "mixed", "aligned", "wide_heads"])
def test_whole_prompt_against_the_plain_statement(made, name, dtype):
    m, cfg, t = made(name, dtype, max_batch=64)
    toks = tokens_for(cfg, 41)
    want = seq_oracle.run(cfg, t, toks)
    s = m.acquire()
    got = m.forward(s, toks, np.arange(len(toks)))
    m.release(s)
    assert err(got, want) < TOL[dtype]


@pytest.mark.parametrize("name", ["mixed", "aligned", "wide_heads"])
def test_residual_stream_after_every_layer(made, name):
    m, cfg, t = made(name, "float32", max_batch=64)
    toks = tokens_for(cfg, 20, seed=5)
    per = []
    seq_oracle.run(cfg, t, toks, per_layer=per)
    m.capture_layers(True)
    s = m.acquire()
    m.forward(s, toks)
    got = m.layers(len(toks))
    m.release(s)
    m.capture_layers(False)
    for i, want in enumerate(per):
        assert np.abs(got[i] - want).max() < 2e-4 * np.abs(want).max(), i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "aligned", "wide_heads"])
def test_token_by_token_and_portions_give_the_whole_prompts_logits(made, name, dtype):
    m, cfg, t = made(name, dtype, max_batch=16)  # 16: a 50-token portion is also cut inside the library
    toks = tokens_for(cfg, 75, seed=2)
    want = seq_oracle.run(cfg, t, toks)
    for sizes in ([1], [2], [3, 1, 7, 2], [50, 2, 23], [16, 17, 15]):
        assert err(run_portions(m, toks, sizes), want) < TOL[dtype], sizes


def test_first_tokens_of_a_sequence(made):
    """sequences shorter than any convolution's taps, alone and as the start of a longer one"""
    m, cfg, t = made("aligned", "float32")
    for n in (1, 2, 3):
        toks = tokens_for(cfg, n, seed=10 + n)
        assert err(run_portions(m, toks, [n]), seq_oracle.run(cfg, t, toks)) < TOL["float32"]
        assert err(run_portions(m, toks, [1]), seq_oracle.run(cfg, t, toks)) < TOL["float32"]


def test_interleaved_requests_and_reused_slots(made):
    m, cfg, t = made("mixed", "float32", max_batch=16)
    seqs = [tokens_for(cfg, n, seed=20 + n) for n in (37, 9, 58)]
    want = [seq_oracle.run(cfg, t, s) for s in seqs]
    sched = seqmodel.RequestScheduler(m)
    got, at = [[] for _ in seqs], [0, 0, 0]
    steps = [5, 2, 11, 1, 3]
    i = 0
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
    # every slot has been used: a new request gets a used one and must start from nothing
    for r in range(4):
        assert err(sched.feed("again", seqs[2], np.arange(len(seqs[2]))), want[2]) < TOL["float32"]
        sched.finish("again")
    with pytest.raises(hip.PSHipError):
        [m.acquire() for _ in range(4)]
    for s in range(3):
        m.release(s)


def peaked_latent_model(window, seed=0, second_layer=True, aligned=False):
    """A latent-attention model whose scores are made by hand: every token's embedding is a constant half (ones) and a token-specific half of
    +-1 (so the norm in front of the mixer changes nothing); queries and the shared rotated key part read the constant half only, so the rotated
    part of the score depends on the DISTANCE alone, 8 (cos(d) + cos(2 pi d / (window - 1))) for window - 1 = 44 k: largest for the token
    itself and for the key at the far edge of the window (44 k is a whole number of turns of the first pair, up to 0.02 rad).  Values read the
    token-specific half.  A key lost or gained at the edge therefore moves the output by a large fraction of itself."""
    rng = np.random.default_rng(seed)
    W, half, V, H, d, dv, qr, kr, dr = 16, 8, 32, 2, 4, 6, 4, 6, 4
    if aligned:  # sizes the matrix-core attention kernels take (the prompt's and the absorbed single-token form); 4 of 16 rotated numbers turn
        d, dv, kr, dr = 16, 8, 16, 16
    f1 = 2 * np.pi / (window - 1)
    mixer = dict(heads=H, dim=d, vdim=dv, q_rank=qr, kv_rank=kr, rot_dim=dr, rot={"base": float(1.0 / f1 ** 2), "dims": 4}, mask={"size": int(window)}, scale=2.0)
    layers = [synth.seq_layer("latent_attention", None, **mixer)] + ([synth.seq_layer("wkv", 24, heads=2, dim=8)] if second_layer else [])
    cfg = synth.seq_config(W, V, layers, taps=1)
    t = synth.seq_tensors(cfg, seed)
    t["embed"] = np.concatenate([np.ones((V, half)), rng.choice([-1.0, 1.0], (V, W - half))], 1).astype(np.float32)
    for n in ("l0.norm1", "l0.canon1"):
        t[n] = np.zeros_like(t[n])
    dq = np.zeros((qr, W), np.float32)
    dq[:, :half] = rng.standard_normal((qr, half)) * 0.5
    t["l0.mix.dq"], t["l0.mix.dq.norm"] = dq, np.ones(qr, np.float32)
    c0 = dq[:, :half].sum(1).astype(np.float64)
    c0 = c0 / np.sqrt(np.mean(c0 * c0) + cfg["norm"]["eps"])       # the query latent of every token
    uq = rng.standard_normal((H, d + dr, qr)) * 0.1
    uq[:, d:, :] = np.outer([2.0, 2.0] + [0.0] * (dr - 2), c0 / (c0 @ c0))   # rotated query part (2, 2, 0, ...) before the rotation
    t["l0.mix.uq"] = uq.reshape(H * (d + dr), qr).astype(np.float32)
    dkv = np.zeros((kr + dr, W), np.float32)
    dkv[:kr, half:] = rng.standard_normal((kr, W - half)) * 0.5     # the latent reads the token-specific half
    dkv[kr:kr + 2, :half] = 2.0 / half                              # shared key part (2, 2, 0, 0) before the rotation
    t["l0.mix.dkv"] = dkv
    t = {k: (f32_to_bf16_bits(np.asarray(v, np.float32)).astype(np.uint32) << 16).view(np.float32).reshape(np.shape(v)) for k, v in t.items()}
    return cfg, t


def _rows(got, want, lo):
    return [err(got[i:i + 1], want[i:i + 1]) for i in range(lo, len(want))]


@pytest.mark.parametrize("aligned", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_edges_in_prompts_and_in_decoding(made, dtype, aligned):
    """The plain statement with a window one shorter loses the edge key and is far off at every later position, one longer gains a key and is
    clearly off; the library agrees with the right one whether the edge passes over prompt tokens, portions' borders or decoded tokens, also
    when the ring of latents (window - 1 + 8 rows here) has wrapped."""
    window = 45
    cfg, t = peaked_latent_model(window, aligned=aligned)
    m, _, _ = made("peaked45%d" % aligned, dtype, max_batch=8, cfg=cfg, tensors=t)
    toks = tokens_for(cfg, 120, seed=3)
    want = seq_oracle.run(cfg, t, toks)
    assert np.median(_rows(seq_oracle.run(cfg, t, toks, window_override={0: window - 1}), want, window - 1)) > 0.3
    assert np.median(_rows(seq_oracle.run(cfg, t, toks, window_override={0: window + 1}), want, window)) > 5e-3
    for sizes in ([120], [1], [8], [5, 2, 12, 1], [43, 1, 1, 1, 1, 1], [44, 2, 1], [46, 1]):
        got = run_portions(m, toks, sizes)
        assert max(_rows(got, want, 0)) < (1e-3 if dtype == "float32" else TOL[dtype]), sizes


@pytest.mark.parametrize("aligned", [False, True])
def test_far_key_among_hundreds_and_a_ring_that_wraps(made, aligned):
    """window 309: the key 308 tokens back carries a large share of the weight.  A 330-token prompt in portions of 64, then 170 single tokens:
    the ring (372 rows) wraps, and the far key is first a prompt token, then a decoded one."""
    window = 309
    cfg, t = peaked_latent_model(window, seed=1, aligned=aligned)
    m, _, _ = made("peaked309%d" % aligned, "float32", max_batch=64, cfg=cfg, tensors=t)
    toks = tokens_for(cfg, 500, seed=4)
    want = seq_oracle.run(cfg, t, toks)
    assert np.median(_rows(seq_oracle.run(cfg, t, toks, window_override={0: window - 1}), want, window - 1)) > 0.1
    s = m.acquire()
    got = [m.forward(s, toks[:330], np.arange(330))] + [m.forward(s, toks[i:i + 1], [0]) for i in range(330, 500)]
    m.release(s)
    assert max(_rows(np.concatenate(got), want, 0)) < 1e-3


def test_long_decoding_keeps_the_recurrent_states(made):
    m, cfg, t = made("mixed", "float32", max_batch=16)
    toks = tokens_for(cfg, 260, seed=6)
    want = seq_oracle.run(cfg, t, toks)
    assert err(run_portions(m, toks, [13, 1, 1, 1, 1, 1, 1, 1]), want) < TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(made, dtype):
    """SeqModel.generate (prefill, then the captured single-token step feeding its own arg-max) picks, at every step, a token whose logit in the
    plain statement is the largest up to rounding; eager launches and a host sampler set to top-1 give the same ids."""
    m, cfg, t = made("mixed", dtype, max_batch=16)
    prompt = tokens_for(cfg, 19, seed=7)
    ids = m.generate(prompt, 24)
    assert ids.shape == (24,)
    full = np.concatenate([prompt, ids])
    want = seq_oracle.run(cfg, t, full[:-1])
    spread = want.max() - want.min()
    for i, tok in enumerate(ids):
        row = want[len(prompt) - 1 + i]
        assert row.max() - row[tok] < (1e-4 if dtype == "float32" else 3e-2) * spread, i
    m.set_mode(1)
    assert np.array_equal(m.generate(prompt, 24), ids)
    m.set_mode(0)
    assert np.array_equal(m.generate(prompt, 24), ids)  # the captured sequence replayed on a slot that was used before
    sm = host.Sampler(host.SamplerCfg.make(cfg["vocab"], seed=1, temperature=1.0, top_p=1.0, top_k=1))
    assert np.array_equal(m.generate(prompt, 24, sampler=sm.sample), ids)
    sm.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_matrix_core_forms_agree_with_the_plain_kernels(made, dtype):
    """mode bit 1 keeps the per-key attention, the expanded single-token step and the 64 x 64 mat-mul: the wide mat-mul, the matrix-core
    attention of a portion and the absorbed single-token attention must give the same logits (fp32: up to the order of sums)"""
    m, cfg, t = made("aligned", dtype, max_batch=64)
    toks = tokens_for(cfg, 150, seed=9)
    fast = [run_portions(m, toks, sizes) for sizes in ([64], [1], [40, 1, 1, 1, 9])]
    m.set_mode(2)
    plain = [run_portions(m, toks, sizes) for sizes in ([64], [1], [40, 1, 1, 1, 9])]
    m.set_mode(0)
    want = seq_oracle.run(cfg, t, toks)
    for a, b in zip(fast, plain):
        assert err(a, b) < (1e-4 if dtype == "float32" else TOL[dtype])
        assert err(a, want) < TOL[dtype]


def test_host_facade_loads_and_generates_the_same(made, tmp_path):
    """load_seq_model of the C++ facade (its own safetensors reader and configuration mapping) over the same files: same ids, same logits"""
    m, cfg, t = made("mixed", "float32", max_batch=16)
    synth.write_seq_model_dir(str(tmp_path), cfg, 0, t)
    assert host.lib().psh_is_seq_model_dir(str(tmp_path).encode()) == 1
    hm = host.HostSeqModel(str(tmp_path), dtype="float32", max_batch=16, n_slots=2)
    prompt = tokens_for(cfg, 19, seed=7)
    ids = m.generate(prompt, 12)
    assert np.array_equal(hm.generate(prompt, 12), ids)
    assert np.array_equal(hm.generate(prompt, 12, host.SamplerCfg.make(cfg["vocab"], seed=3, temperature=1.0, top_p=1.0, top_k=1)), ids)
    s, s2 = hm.acquire(), m.acquire()
    a, b = hm.forward(s, prompt, [0, 5, 18]), m.forward(s2, prompt, [0, 5, 18])
    hm.release(s)
    m.release(s2)
    assert np.array_equal(a, b)
    with pytest.raises(host.HostError):
        host.HostModel(str(tmp_path))  # the quantized path's loader says what this folder is instead of looking for model.json
    hm.close()


def test_refusals(ctx, tmp_path):
    cfg = dict(CONFIGS["wkv"])
    synth.write_seq_model_dir(str(tmp_path), cfg, 0)
    m = seqmodel.load_model(ctx, str(tmp_path), dtype="float32", max_batch=4, n_slots=1)
    s = m.acquire()
    with pytest.raises(hip.PSHipError):
        m.forward(s, [cfg["vocab"]])
    with pytest.raises(hip.PSHipError):
        m.forward(s + 1, [0])
    m.release(s)
    with pytest.raises(hip.PSHipError):
        m.release(s)
    m.close()
