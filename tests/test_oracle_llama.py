"""Pins the C checker (oracle/llama2_oracle.c) against library routines and an
independent library implementation of the Llama-2 architecture.  CPU only."""
import numpy as np
import pytest

from oracle import llama2 as O

TINY = dict(dim=48, hidden_dim=128, n_layers=3, n_heads=6, n_kv_heads=6, vocab_size=200, seq_len=32)
TINY_GQA = dict(dim=48, hidden_dim=96, n_layers=2, n_heads=6, n_kv_heads=2, vocab_size=120, seq_len=24)


def test_softmax_vs_scipy():
    from scipy.special import softmax
    x = np.random.default_rng(0).standard_normal(777).astype(np.float32) * 4
    assert np.allclose(O.softmax(x), softmax(x.astype(np.float64)), rtol=2e-6, atol=1e-9)
    assert O.softmax(np.float32([3.0]))[0] == 1.0


def test_rmsnorm_vs_torch():
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(1)
    x = rng.standard_normal(288).astype(np.float32)
    w = rng.standard_normal(288).astype(np.float32)
    ref = F.rms_norm(torch.from_numpy(x).double(), (288,), torch.from_numpy(w).double(), eps=1e-5).numpy()
    assert np.allclose(O.rmsnorm(x, w), ref, rtol=3e-6, atol=1e-7)


def test_matvec_vs_numpy_and_row_major_layout():
    rng = np.random.default_rng(2)
    w = rng.standard_normal((37, 53)).astype(np.float32)
    x = rng.standard_normal(53).astype(np.float32)
    assert np.allclose(O.matvec(w, x), w.astype(np.float64) @ x, rtol=1e-5, atol=1e-5)
    e = np.zeros(53, np.float32)
    e[7] = 1
    assert np.array_equal(O.matvec(w, e), w[:, 7])


def test_freq_tables_and_rope_closed_form():
    hs, S, H = 16, 40, 3
    c, s = O.freq_tables(hs, S)
    j = np.arange(hs // 2)
    ang = np.arange(S)[:, None] * 10000.0 ** (-2.0 * j / hs)[None, :]
    assert np.allclose(c, np.cos(ang), atol=3e-6) and np.allclose(s, np.sin(ang), atol=3e-6)
    rng = np.random.default_rng(3)
    q = rng.standard_normal((H, hs)).astype(np.float32)
    k = rng.standard_normal((H, hs)).astype(np.float32)
    for pos in (0, 1, 17, 39):
        q2, k2 = O.rope_pairs(q, k, c, s, pos)
        for src, out in ((q, q2), (k, k2)):
            z = (src[:, 0::2] + 1j * src[:, 1::2]) * np.exp(1j * ang[pos])[None, :]
            assert np.allclose(out[:, 0::2], z.real, atol=1e-5)
            assert np.allclose(out[:, 1::2], z.imag, atol=1e-5)
    q0, k0 = O.rope_pairs(q, k, c, s, 0)
    assert np.array_equal(q0, q) and np.array_equal(k0, k)


def test_argmax_first_max_wins():
    assert O.argmax(np.float32([1, 5, 5, 2])) == 1
    assert O.argmax(np.float32([-3, -3, -3])) == 0
    assert O.argmax(np.float32([0, 1, 2, 9])) == 3


def _hf_model(cfg, views, shared):
    import torch
    from transformers import LlamaConfig, LlamaForCausalLM
    hc = LlamaConfig(hidden_size=cfg["dim"], intermediate_size=cfg["hidden_dim"],
                     num_hidden_layers=cfg["n_layers"], num_attention_heads=cfg["n_heads"],
                     num_key_value_heads=cfg["n_kv_heads"], vocab_size=cfg["vocab_size"],
                     max_position_embeddings=cfg["seq_len"], rms_norm_eps=1e-5, rope_theta=10000.0,
                     tie_word_embeddings=False, attention_bias=False, mlp_bias=False)
    hc._attn_implementation = "eager"
    m = LlamaForCausalLM(hc).double().eval()
    hs = cfg["dim"] // cfg["n_heads"]
    # adjacent-pair rotary -> half-split rotary: reorder q/k output rows inside each head
    perm = np.concatenate([np.arange(0, hs, 2), np.arange(1, hs, 2)])

    def rot(w, nh):
        return w.reshape(nh, hs, -1)[:, perm, :].reshape(nh * hs, -1)

    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).double()
    sd = {"model.embed_tokens.weight": t(views["tok_emb"]), "model.norm.weight": t(views["rms_final"]),
          "lm_head.weight": t(views["tok_emb"] if shared else views["wcls"])}
    for l in range(cfg["n_layers"]):
        p = "model.layers.%d." % l
        sd[p + "input_layernorm.weight"] = t(views["rms_att"][l])
        sd[p + "post_attention_layernorm.weight"] = t(views["rms_ffn"][l])
        sd[p + "self_attn.q_proj.weight"] = t(rot(views["wq"][l], cfg["n_heads"]))
        sd[p + "self_attn.k_proj.weight"] = t(rot(views["wk"][l], cfg["n_kv_heads"]))
        sd[p + "self_attn.v_proj.weight"] = t(views["wv"][l])
        sd[p + "self_attn.o_proj.weight"] = t(views["wo"][l])
        sd[p + "mlp.gate_proj.weight"] = t(views["w1"][l])
        sd[p + "mlp.down_proj.weight"] = t(views["w2"][l])
        sd[p + "mlp.up_proj.weight"] = t(views["w3"][l])
    missing = m.load_state_dict(sd, strict=False)
    assert not [k for k in missing.missing_keys if "rotary" not in k], missing
    return m


@pytest.mark.parametrize("cfg,shared", [(TINY, False), (TINY, True), (TINY_GQA, False)])
def test_forward_vs_transformers_llama(cfg, shared):
    """Incremental KV-cache decode of the checker == full-sequence forward of
    transformers.LlamaForCausalLM (fp64) on the same weights, every position."""
    import torch
    blob, views = O.random_weights(cfg, seed=11, shared_classifier=shared, std=0.2)
    # non-trivial norm weights so a dropped weight multiply would show
    rng = np.random.default_rng(5)
    for k in ("rms_att", "rms_ffn", "rms_final"):
        views[k][...] = 1.0 + 0.3 * rng.standard_normal(views[k].shape).astype(np.float32)
    toks = rng.integers(0, cfg["vocab_size"], 20)
    m = O.Llama(cfg, blob, shared)
    mine = np.stack([m.forward(int(t), i) for i, t in enumerate(toks)])
    hf = _hf_model(cfg, views, shared)
    with torch.no_grad():
        ref = hf(torch.from_numpy(toks)[None]).logits[0].numpy()
    err = np.abs(mine - ref).max() / np.abs(ref).max()
    assert err < 2e-5, err
    assert np.array_equal(mine.argmax(-1), ref.argmax(-1))


def test_generate_greedy_feeds_back_argmax_and_is_deterministic():
    blob, _ = O.random_weights(TINY, seed=3, std=0.2)
    m = O.Llama(TINY, blob)
    prompt = np.array([5, 17, 3, 99], np.int32)
    ids, lg = m.generate_greedy(prompt, 24, want_logits=True)
    assert np.array_equal(ids, lg.argmax(-1))
    m2 = O.Llama(TINY, blob)
    seq = list(prompt)
    for pos in range(24):
        tok = seq[pos] if pos < len(prompt) else int(ids[pos - 1])
        l2 = m2.forward(tok, pos)
        assert np.array_equal(l2, lg[pos])
    assert np.array_equal(O.Llama(TINY, blob).generate_greedy(prompt, 24), ids)


def test_checkpoint_v1_header(tmp_path):
    import struct
    blob, _ = O.random_weights(TINY, seed=1)
    p = tmp_path / "m.bin"
    O.write_checkpoint_v1(str(p), TINY, blob, shared_classifier=False)
    raw = p.read_bytes()
    assert struct.unpack("<Ii", raw[:8]) == (0x616B3432, 1)
    assert struct.unpack("<7i", raw[8:36]) == tuple(TINY[k] for k in O.CONFIG_FIELDS)
    assert raw[36] == 0 and len(raw) == 256 + blob.size * 4
    assert np.array_equal(np.frombuffer(raw[256:], np.float32), blob)


# ---- sampler (llama2_sampler.cpp) -------------------------------------------------------------------

def _xorshift64star(state):
    """xorshift64* on Python integers (unbounded, masked to 64 bits): an independent arithmetic for the same recurrence."""
    M = (1 << 64) - 1
    state ^= state >> 12
    state ^= (state << 25) & M
    state ^= state >> 27
    return state, ((state * 0x2545F4914F6CDD1D) & M) >> 32


def test_rng_recurrence_range_and_uniformity():
    # worked by hand for state 1: no bit reaches the >> shifts, so the new state is 1 | 1 << 25
    s = O.Sampler(1.0, 0.9, 1)
    assert s.random_u32() == ((33554433 * 0x2545F4914F6CDD1D) & ((1 << 64) - 1)) >> 32
    assert s.state.value == 33554433
    for seed in (1, 2, 1234567, 0xDEADBEEFCAFEF00D):
        s = O.Sampler(1.0, 0.9, seed)
        st = seed
        for _ in range(200):
            st, u = _xorshift64star(st)
            assert s.random_u32() == u and s.state.value == st
    s = O.Sampler(1.0, 0.9, 0)            # the all-zero state is a fixed point: every coin is 0
    assert s.random_u32() == 0 and s.random_f32() == 0.0
    s = O.Sampler(1.0, 0.9, 42)
    f = np.array([s.random_f32() for _ in range(100000)])
    assert f.min() >= 0.0 and f.max() < 1.0
    assert np.all(f * 16777216 == np.floor(f * 16777216))            # 24-bit coins
    hist = np.bincount((f * 16).astype(int), minlength=16)
    chi2 = ((hist - 6250.0) ** 2 / 6250.0).sum()
    assert chi2 < 45                                                    # 15 degrees of freedom, p ~ 1e-4


def test_sample_mult_is_the_inverse_cdf():
    rng = np.random.default_rng(7)
    for n in (2, 17, 1000):
        p = rng.random(n).astype(np.float32)
        p /= p.sum()
        cdf = np.cumsum(p.astype(np.float64))
        for coin in rng.random(300):
            j = int(np.searchsorted(cdf, coin, side="right"))
            if j < n and min(abs(cdf - coin)) > 1e-5:                   # away from the rounding of the boundaries
                assert O.sample_mult(p, coin) == j
        assert O.sample_mult(p, 0.0) == 0
        assert O.sample_mult(p, 1.5) == n - 1                           # past the end: the last index
    p = np.array([0, 0, 0.5, 0.5], np.float32)
    assert O.sample_mult(p, 0.0) == 2                                   # strict '<': zero-probability entries are skipped


def test_sample_topp_nucleus_and_frequencies():
    rng = np.random.default_rng(8)
    n, topp = 50, 0.8
    p = rng.random(n).astype(np.float32) ** 4
    p /= p.sum()
    order = np.argsort(-p.astype(np.float64), kind="stable")
    cum = np.cumsum(p[order].astype(np.float64))
    k = int(np.searchsorted(cum, topp, side="right")) + 1               # smallest prefix whose mass exceeds topp
    nucleus = set(order[:k].tolist())
    coins = (np.arange(20000) + 0.5) / 20000                            # a regular grid of coins = exact quantiles
    got = np.array([O.sample_topp(p, topp, c) for c in coins])
    assert set(got.tolist()) == nucleus
    freq = np.bincount(got, minlength=n) / len(coins)
    want = np.zeros(n)
    want[order[:k]] = p[order[:k]] / cum[k - 1]
    assert np.abs(freq - want).max() < 2e-4                             # grid resolution 5e-5 per boundary
    # a nucleus of one token: always the most likely one; probabilities below (1-topp)/(n-1) never appear
    assert all(O.sample_topp(p, 1e-6, c) == order[0] for c in (0.0, 0.3, 0.999))
    cut = (1 - topp) / (n - 1)
    assert all(p[i] >= cut for i in set(got.tolist()))


def test_sample_temperature_softmax_and_random_stream():
    rng = np.random.default_rng(9)
    logits = (rng.standard_normal(64) * 2).astype(np.float32)
    assert O.Sampler(0.0, 0.9, 5).sample(logits) == int(logits.argmax())          # temperature 0: greedy, no coin drawn
    s = O.Sampler(0.0, 0.9, 5)
    s.sample(logits)
    assert s.state.value == 5
    assert all(O.Sampler(1e-3, 0.0, seed).sample(logits) == int(logits.argmax()) for seed in range(1, 20))
    T = 0.7
    s = O.Sampler(T, 0.0, 99)                                                        # topp <= 0: plain multinomial
    draws = np.array([s.sample(logits) for _ in range(40000)])
    z = logits.astype(np.float64) / T
    want = np.exp(z - z.max())
    want /= want.sum()
    freq = np.bincount(draws, minlength=64) / len(draws)
    assert np.abs(freq - want).max() < 4 * np.sqrt(want.max() / len(draws)) + 1e-3
    # one coin per call, taken from the same stream as random_f32
    a, b = O.Sampler(T, 0.0, 7), O.Sampler(T, 0.0, 7)
    p = np.exp((logits / np.float32(T)) - (logits / np.float32(T)).max())
    for _ in range(50):
        coin = b.random_f32()
        tok = a.sample(logits)
        assert a.state.value == b.state.value
        pf = (p / p.sum(dtype=np.float32)).astype(np.float32)
        cdf = np.cumsum(pf.astype(np.float64))
        if min(abs(cdf - coin)) > 1e-5:
            assert tok == int(np.searchsorted(cdf, coin, side="right"))


def test_generate_sampled_loop_draws_a_coin_at_every_position():
    blob, _ = O.random_weights(TINY, seed=3, std=0.2)
    prompt = np.array([5, 17, 3, 99], np.int32)
    greedy = O.Llama(TINY, blob).generate_greedy(prompt, 24)
    assert np.array_equal(O.Llama(TINY, blob).generate_sampled(prompt, 24, O.Sampler(0.0, 0.9, 11)), greedy)
    for topp in (0.9, 0.0):
        ids = O.Llama(TINY, blob).generate_sampled(prompt, 24, O.Sampler(0.8, topp, 11))
        assert np.array_equal(ids, O.Llama(TINY, blob).generate_sampled(prompt, 24, O.Sampler(0.8, topp, 11)))
        assert not np.array_equal(ids, greedy)
        # step by step: forward, then one sample() per position, the prompt positions included
        m, s = O.Llama(TINY, blob), O.Sampler(0.8, topp, 11)
        nxt = 0
        for pos in range(24):
            tok = int(prompt[pos]) if pos < len(prompt) else nxt
            nxt = s.sample(m.forward(tok, pos))
            assert nxt == ids[pos]


def test_package_checkpoint_writer_matches_the_checkers(tmp_path):
    """The benchmark writes its synthetic model with the package's own writer; the file and the weights are the ones
    the checker's writer gives for the same seed, so both sides load the same model."""
    from mycaffe_amd import checkpoint as C
    cfg = dict(dim=64, hidden_dim=172, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=256, seq_len=32)
    for shared in (False, True):
        a, _ = O.random_weights(cfg, seed=3, shared_classifier=shared, std=0.2)
        b = C.random_model(cfg, 3, shared_classifier=shared, std=0.2)
        assert np.array_equal(a, b)
        pa, pb = str(tmp_path / "a.bin"), str(tmp_path / "b.bin")
        O.write_checkpoint_v1(pa, cfg, a, shared)
        C.write_v1(pb, cfg, b, shared)
        assert open(pa, "rb").read() == open(pb, "rb").read()


def test_bf16_rounding_vs_torch():
    import torch
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(4096).astype(np.float32) * 10.0 ** rng.integers(-30, 30, 4096).astype(np.float32),
        # exact ties between two bfloat16 neighbours, even and odd kept bit below them
        np.array([0x3f808000, 0x3f818000, 0xbf808000, 0xbf818000, 0x00008000, 0x00018000, 0x7f7f8000, 0x7f7fffff],
                 np.uint32).view(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-40, 3.3895314e38], np.float32),
    ])
    with np.errstate(over="ignore"):
        ref = torch.from_numpy(x.copy()).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(O.round_bf16(x).view(np.uint32), ref.view(np.uint32))
    assert np.isnan(O.round_bf16(np.array([np.nan], np.float32))[0])


@pytest.mark.parametrize("cfg", [TINY, TINY_GQA], ids=["mha", "gqa"])
def test_bf16_cache_option_vs_a_forward_assembled_from_the_pinned_routines(cfg):
    """The checker-only 16-bit cache option: the same logits as a forward written out here from the individually pinned
    routines (rmsnorm, matvec, rope, softmax) with torch doing the rounding of every key and value that enters the cache."""
    import torch
    blob, w = O.random_weights(cfg, seed=5, std=0.3)
    dim, H, kvH = cfg["dim"], cfg["n_heads"], cfg["n_kv_heads"]
    hs, L = dim // H, cfg["n_layers"]
    fcos, fsin = O.freq_tables(hs, cfg["seq_len"])
    rnd = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(torch.bfloat16).to(torch.float32).numpy()
    toks = [3, 77, 12, 5, 41, 9]
    kc = [[] for _ in range(L)]
    vc = [[] for _ in range(L)]
    mine = []
    for pos, tok in enumerate(toks):
        x = w["tok_emb"][tok].copy()
        for l in range(L):
            xb = O.rmsnorm(x, w["rms_att"][l])
            q = O.matvec(w["wq"][l], xb).reshape(H, hs)
            k = O.matvec(w["wk"][l], xb).reshape(kvH, hs)
            v = O.matvec(w["wv"][l], xb).reshape(kvH, hs)
            # the checker rotates q and k in one call over n_heads heads of which the first kv heads are k's
            kpad = np.zeros((H, hs), np.float32)
            kpad[:kvH] = k
            q, kpad = O.rope_pairs(q, kpad, fcos, fsin, pos)
            kc[l].append(rnd(kpad[:kvH]))
            vc[l].append(rnd(v))
            o = np.zeros((H, hs), np.float32)
            for h in range(H):
                g = h // (H // kvH)
                s = np.stack([kc[l][t][g] for t in range(pos + 1)]).astype(np.float64) @ q[h].astype(np.float64) / np.sqrt(hs)
                a = O.softmax(s.astype(np.float32))
                o[h] = (a[:, None].astype(np.float64) * np.stack([vc[l][t][g] for t in range(pos + 1)])).sum(0)
            x = x + O.matvec(w["wo"][l], o.ravel())
            xb = O.rmsnorm(x, w["rms_ffn"][l])
            h1 = O.matvec(w["w1"][l], xb)
            h3 = O.matvec(w["w3"][l], xb)
            x = x + O.matvec(w["w2"][l], (h1 / (1.0 + np.exp(-h1)) * h3).astype(np.float32))
        x = O.rmsnorm(x, w["rms_final"])
        mine.append(O.matvec(w.get("wcls", w["tok_emb"]), x))
    O.set_kv_bf16(True)
    try:
        m = O.Llama(cfg, blob)
        got = np.stack([m.forward(t, p) for p, t in enumerate(toks)])
    finally:
        O.set_kv_bf16(False)
    plain = np.stack([O.Llama(cfg, blob).forward(t, p) for p, t in enumerate(toks)][:1])
    mine = np.stack(mine)
    assert np.abs(got - mine).max() / np.abs(mine).max() < 2e-5
    # the option changes the result (position 0 attends over its own rounded value) and is off again afterwards
    assert np.abs(got[0] - plain[0]).max() > 1e-6
    assert np.array_equal(O.Llama(cfg, blob).forward(toks[0], 0), plain[0])
