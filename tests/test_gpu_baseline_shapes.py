"""Parity at the exact shapes the benchmark quotes its figures on (the five benchmark configurations), each
against the CPU checker:

* 110M-shape Llama (dim 768, 12 layers, 12 x 64, ffn 2048, vocabulary 32000, context 1024): batch 1 fp32 logits and
  ids, batch 16 = 16 independent CPU runs, bf16 weight storage against the checker on bf16-rounded weights;
* decode attention at 32 heads x 128 over a cache of 4096 positions, batch 1 and 32, fp32 and bf16, with and without
  the rotate-and-append step;
* encoder / decoder / cross attention of the d_model 512, 8 x 64, batch 32, 256 / 128 configuration in bf16;
* the InnerProduct GEMMs 8192 x 2304 x 768 and 8192 x 768 x 768 in fp32 and bf16, and the whole causal self attention
  layer at B = 8, T = 1024, C = 768.
"""
import numpy as np
import pytest

from mycaffe_amd.cudadnn import CudaDnn
from mycaffe_amd.layers import Blob, CausalSelfAttentionLayer, MultiheadAttentionLayer
from mycaffe_amd.llm_inference import LlmInference
from oracle import attention_ref as R
from oracle import llama2 as O
from tests.conftest import BF16_RTOL, FP32_RTOL, assert_close, bf16_round

pytestmark = pytest.mark.gpu

C4 = dict(dim=768, hidden_dim=2048, n_layers=12, n_heads=12, n_kv_heads=12, vocab_size=32000, seq_len=1024)


# ---- 110M-shape Llama ------------------------------------------------------------------------

@pytest.fixture(scope="module")
def c4_model(tmp_path_factory):
    blob, _ = O.random_weights(C4, seed=1, shared_classifier=False, std=0.02)
    path = str(tmp_path_factory.mktemp("c4") / "llama110m.bin")
    O.write_checkpoint_v1(path, C4, blob, False)
    return path, blob


@pytest.fixture()
def llm():
    cuda = CudaDnn(0)
    inf = LlmInference(cuda)
    inf.Initialize(fTemperature=0.0)
    yield inf
    inf.CleanUp()
    cuda.Dispose()


def _first_max(logits):
    """sample_argmax (llama2_sampler.cpp:25-36): strict '>' scan, so the lowest index wins a tie."""
    return np.argmax(logits, axis=-1)


def _ids_match(ids, ref_ids, ref_logits, what, logits=None):
    """Greedy ids bit-exact against the checker.  Sequences can only part where the checker's own top-2 logits are
    closer than the fp32 parity tolerance allows the two implementations to differ: anything else fails.  When the
    device logits are given, every chosen id must also be the first-max argmax of those logits, bit-exact."""
    ids, ref_ids = np.asarray(ids), np.asarray(ref_ids)
    if logits is not None:
        assert np.array_equal(ids, _first_max(logits)), what + ": id is not the first-max argmax of the device logits"
    if np.array_equal(ids, ref_ids):
        return True
    first = int(np.argmax(ids != ref_ids))
    top2 = np.sort(ref_logits[first])[-2:]
    gap = (top2[1] - top2[0]) / max(float(np.abs(ref_logits[first]).max()), 1e-30)
    print("%s: ids part at step %d, checker's relative top-2 gap %.3e" % (what, first, gap), flush=True)
    assert gap < FP32_RTOL, "%s: ids differ at step %d where the checker's top-2 gap is %.3e" % (what, first, gap)
    return False


def _batch_rows_against_cpu(cpu, prompts, n, ids, logits, what):
    """Every sequence of a batched generation against its own CPU run: logits of every step up to the point where the
    two id streams part (they may only part at a tie of the checker's top-2 logits), ids bit-exact before it."""
    parted = 0
    for b in range(len(prompts)):
        ref_ids, ref_logits = cpu.generate_greedy(prompts[b], n, want_logits=True)
        same = _ids_match(ids[b], ref_ids, ref_logits, "%s, sequence %d" % (what, b), logits[b])
        upto = n if same else int(np.argmax(np.asarray(ids[b]) != np.asarray(ref_ids))) + 1
        assert_close(logits[b, :upto], ref_logits[:upto], FP32_RTOL, "%s, sequence %d logits" % (what, b))
        parted += 0 if same else 1
    assert parted <= 2, "%s: %d of %d sequences parted from the checker" % (what, parted, len(prompts))


def test_llama110m_batch1_fp32_logits_and_ids(llm, c4_model):
    path, blob = c4_model
    llm.Load(path)
    prompt = np.random.default_rng(1).integers(3, C4["vocab_size"], 128)
    n = 200   # 128 forced prompt positions, then 72 greedy ones
    ref_ids, ref_logits = O.Llama(C4, blob).generate_greedy(prompt, n, want_logits=True)
    ids, logits = llm.GenerateIds(prompt, n, want_logits=True)   # eager launches
    assert_close(logits, ref_logits, FP32_RTOL, "110M logits, every position")
    assert _ids_match(ids, ref_ids, ref_logits, "110M eager", logits)
    ids_graph = llm.GenerateIds(prompt, n)                        # one captured graph per step
    assert llm.LastRunUsedGraph()
    assert np.array_equal(ids_graph, ids)
    # the 128 prompt positions went through the batched pass; one decode step per position gives the same
    assert llm.LastPrefill()[1] == 128
    llm.SetOption(7, 0)
    ids_loop, logits_loop = llm.GenerateIds(prompt, n, want_logits=True)
    assert llm.LastPrefill() == (0.0, 0)
    assert_close(logits_loop, ref_logits, FP32_RTOL, "110M logits, one step per prompt position")
    assert np.array_equal(ids_loop, ids)


def test_llama110m_batch1_fp32_whole_generation_to_1024_positions(llm, c4_model):
    # benchmark configuration 4 at its full length: 128 forced ids, then greedy to position 1023 (cache rows beyond the
    # first split iteration, every split of the fused decode attention in use)
    path, blob = c4_model
    llm.Load(path)
    prompt = np.random.default_rng(4).integers(3, C4["vocab_size"], 128)
    n = C4["seq_len"]
    ref_ids, ref_logits = O.Llama(C4, blob).generate_greedy(prompt, n, want_logits=True)
    ids, logits = llm.GenerateIds(prompt, n, want_logits=True)   # eager launches
    same = _ids_match(ids, ref_ids, ref_logits, "110M to 1024 positions", logits)
    upto = n if same else int(np.argmax(np.asarray(ids) != np.asarray(ref_ids))) + 1
    assert upto > 900, "ids part from the checker at position %d" % upto
    assert_close(logits[:upto], ref_logits[:upto], FP32_RTOL, "110M logits up to position %d" % upto)
    ids_graph = llm.GenerateIds(prompt, n)                        # replays of the captured step
    assert llm.LastRunUsedGraph()
    assert np.array_equal(ids_graph, ids)


def test_llama110m_batch16_fp32_every_row_an_independent_cpu_run(llm, c4_model):
    path, blob = c4_model
    llm.Load(path)
    rng = np.random.default_rng(16)
    B, nP, n = 16, 24, 64
    prompts = rng.integers(3, C4["vocab_size"], (B, nP))
    ids, logits = llm.GenerateBatch(prompts, n, want_logits=True)   # eager launches
    ids_graph = llm.GenerateBatch(prompts, n)                        # one captured graph per step
    assert llm.LastRunUsedGraph()
    assert np.array_equal(ids_graph, ids)
    _batch_rows_against_cpu(O.Llama(C4, blob), prompts, n, ids, logits, "110M batch 16")


@pytest.mark.parametrize("batch", [1, 16])
def test_llama110m_bf16_weights_against_checker_on_rounded_weights(llm, c4_model, batch):
    path, blob = c4_model
    llm.SetOption(1, 1)
    llm.Load(path)
    rb = bf16_round(blob)
    cpu = O.Llama(C4, rb)
    rng = np.random.default_rng(5 + batch)
    if batch == 1:
        prompt = rng.integers(3, C4["vocab_size"], 128)
        n = 176
        ref_ids, ref_logits = cpu.generate_greedy(prompt, n, want_logits=True)
        ids, logits = llm.GenerateIds(prompt, n, want_logits=True)
        assert_close(logits, ref_logits, FP32_RTOL, "bf16-weight logits vs checker on rounded weights")
        assert _ids_match(ids, ref_ids, ref_logits, "110M bf16 weights", logits)
        assert np.array_equal(llm.GenerateIds(prompt, n), ids)
        # and the rounding itself stays inside the 16-bit bar against the fp32 model
        _, full = O.Llama(C4, blob).generate_greedy(prompt, 4, want_logits=True)
        assert_close(logits[:4], full, BF16_RTOL, "bf16 weights vs fp32 model")
    else:
        prompts = rng.integers(3, C4["vocab_size"], (batch, 16))
        n = 48
        ids, logits = llm.GenerateBatch(prompts, n, want_logits=True)
        assert np.array_equal(llm.GenerateBatch(prompts, n), ids)
        _batch_rows_against_cpu(cpu, prompts, n, ids, logits, "110M bf16 batch 16")


def test_llama110m_batch16_bf16_weights_and_bf16_cache(llm, c4_model):
    """The fully 16-bit-storage configuration at the benchmarked shape: bf16 weights and bf16 key / value caches, batch 16,
    a 128-token prompt per sequence (the batched prompt pass through the GEMM path) and greedy steps after it.  Every row
    against its own CPU run on the rounded weights with the checker's cache rounding; 3e-3 on the logits: a last-bit
    difference between the two sides' fp32 key or value next to a rounding boundary moves the cached element by one
    bfloat16 step, and a sequence caches 3 million elements here (2 x 12 layers x 768 x 160 positions)."""
    path, blob = c4_model
    llm.SetOption(1, 1)
    llm.SetOption(8, 1)
    llm.Load(path)
    rb = bf16_round(blob)
    rng = np.random.default_rng(77)
    B, nP, n = 16, 128, 160
    prompts = rng.integers(3, C4["vocab_size"], (B, nP))
    ids, logits = llm.GenerateBatch(prompts, n, want_logits=True)
    assert llm.LastPrefill()[1] == B * nP
    assert np.array_equal(llm.GenerateBatch(prompts, n), ids)
    assert llm.LastRunUsedGraph()
    O.set_kv_bf16(True)
    try:
        cpu = O.Llama(C4, rb)
        parted = 0
        for b in range(0, B, 3):   # six of the sixteen rows: 160 positions of the 110M model take the CPU a second each
            ref_ids, ref_logits = cpu.generate_greedy(prompts[b], n, want_logits=True)
            assert np.array_equal(ids[b], _first_max(logits[b]))
            same = np.array_equal(ids[b], ref_ids)
            upto = n if same else int(np.argmax(ids[b] != ref_ids)) + 1
            assert_close(logits[b, :upto], ref_logits[:upto], 3e-3, "110M 16-bit weights and caches, sequence %d" % b)
            if not same:
                top2 = np.sort(ref_logits[upto - 1])[-2:]
                assert (top2[1] - top2[0]) / np.abs(ref_logits[upto - 1]).max() < 3e-3, "sequence %d parts at a decisive step" % b
                parted += 1
        # Every parting above was at a step the checker itself decides by less than the bar.  How many rows part depends on
        # how many cached elements sit next to a rounding boundary: the prompt pass multiplies its activations as two
        # bf16 numbers each (sixteen leading bits), so its keys and values differ from the checker's in the last bits.
        assert parted <= 3
    finally:
        O.set_kv_bf16(False)


def test_llama110m_batch16_bf16_weights_prompt_pass_with_bf16_activations(llm, c4_model):
    """Option 10: the batched prompt pass over bf16 weights with its activations rounded to bf16 and the attention in
    bf16 (one pass over each weight matrix on the bf16 matrix cores instead of two).  16 sequences x 128 prompt tokens.
    The logits of every prompt position stay within the 16-bit bar of the checker on the rounded weights (which keeps fp32
    activations), an id may differ only where the checker's top-2 logits are closer than that bar, and the default
    (option 10 = 0) stays within the fp32 bar on the same prompts."""
    path, blob = c4_model
    llm.SetOption(1, 1)
    llm.Load(path)
    cpu = O.Llama(C4, bf16_round(blob))
    rng = np.random.default_rng(31)
    B, nP, n = 16, 128, 132
    prompts = rng.integers(3, C4["vocab_size"], (B, nP))
    llm.SetOption(10, 1)
    ids16, logits16 = llm.GenerateBatch(prompts, n, want_logits=True)
    assert llm.LastPrefill()[1] == B * nP
    llm.SetOption(10, 0)
    ids, logits = llm.GenerateBatch(prompts, n, want_logits=True)
    assert llm.LastPrefill()[1] == B * nP
    for b in range(0, B, 5):
        ref_ids, ref_logits = cpu.generate_greedy(prompts[b], n, want_logits=True)
        assert_close(logits[b], ref_logits, FP32_RTOL, "two bf16 numbers per activation, sequence %d" % b)
        assert np.array_equal(ids16[b], _first_max(logits16[b]))
        # ids of prompt positions are not fed back; from the last prompt position on a different id parts the two runs
        diff = [t for t in np.nonzero(ids16[b] != ref_ids)[0]]
        late = [t for t in diff if t >= nP - 1]
        upto = n if not late else late[0] + 1
        assert_close(logits16[b, :upto], ref_logits[:upto], BF16_RTOL, "bf16 activations, sequence %d" % b)
        for t in [t for t in diff if t < upto]:
            top2 = np.sort(ref_logits[t])[-2:]
            assert (top2[1] - top2[0]) / np.abs(ref_logits[t]).max() < BF16_RTOL, "sequence %d: id differs at a decisive step %d" % (b, t)


@pytest.mark.parametrize("topp", [0.9, 0.0, 0.3])
def test_llama110m_device_sampler_against_the_host_sampler_at_vocab_32000(c4_model, topp):
    """Temperature 0.8 at the 110M shape (32000 logits a step): the device sampler (option 11 = 1, default: one kernel per
    step, the steps replayed as a captured graph) against the host sampler after a copy of the logits (option 11 = 0, the
    reference's arrangement, itself checked against the C checker in test_gpu_llama.py).  Same seed, same coin stream;
    single sequence and a batch of three; the second generation continues the stream of the first.  An id may differ only
    where the coin lies within rounding of an edge of the cumulative distribution: none does for these seeds.  Both runs
    take the prompt one position per step (option 7 = 0), so that the two samplers see the same logits bit for bit: a
    random model's 32000 probabilities are nearly equal, and the last bit of a logit - the batched prompt pass sums in
    another order - moves such a draw to a neighbouring id."""
    path, _ = c4_model
    rng = np.random.default_rng(12)
    prompt = rng.integers(3, C4["vocab_size"], 9)
    prompts = rng.integers(3, C4["vocab_size"], (3, 9))
    out = {}
    for dev in (0, 1):
        cuda = CudaDnn(0)
        inf = LlmInference(cuda)
        inf.Initialize(fTemperature=0.8, fTopp=topp, lSeed=4242)
        inf.SetOption(5, 1)
        inf.SetOption(7, 0)
        inf.SetOption(11, dev)
        inf.Load(path)
        a = inf.GenerateIds(prompt, 60)
        graph = inf.LastRunUsedGraph()
        b = inf.GenerateIds(prompt, 40)          # continues the random stream
        c = inf.GenerateBatch(prompts, 30)
        out[dev] = (a, b, c)
        assert graph                             # either way the step's kernels replay as a graph; the host path stops at the logits
        inf.CleanUp()
        cuda.Dispose()
    for x, y in zip(out[0], out[1]):
        assert np.array_equal(x, y)
    assert not np.array_equal(out[1][0][:40], out[1][1])   # a different stretch of the stream, a different text


def test_weight_storage_option_after_load_leaves_the_loaded_model_alone(llm, c4_model):
    # option 1 names the storage of the NEXT load: flipping it on a loaded fp32 model changes nothing
    path, blob = c4_model
    llm.Load(path)
    prompt = np.random.default_rng(3).integers(3, C4["vocab_size"], 8)
    ids = llm.GenerateIds(prompt, 24)
    llm.SetOption(1, 1)
    assert np.array_equal(llm.GenerateIds(prompt, 24), ids)
    ref_ids, ref_logits = O.Llama(C4, blob).generate_greedy(prompt, 24, want_logits=True)
    assert _ids_match(ids, ref_ids, ref_logits, "fp32 model after the option flip")


# ---- fused causal attention at the long-context shape of the benchmark ---------------------------

def test_flash_attention_bf16_B4_T4096_32x128_causal_sampled_heads(dev):
    """The Llama-2 7B head shape at full context (the second prefill target of the bench line): the software-pipelined
    kernel with the grouped head order (K and V of the 128 heads are 268 MB).  Three (batch, head) pairs against the fp64
    closed form, and the heads between them against a cheap invariant (row 0 of a causal head returns V[0])."""
    B, H, T, hs = 4, 32, 4096, 128
    rng = np.random.default_rng(40)
    blk = bf16_round(rng.standard_normal((3, T, hs)).astype(np.float32))
    picks = [(0, 0), (1, 17), (3, 31)]
    n = B * H * T * hs
    hq, hk, hv, hy = (dev.zeros(n, True) for _ in range(4))
    # every head gets seeded data cheaply: one random block copied on the device, the picked heads their own q, k, v
    fill = bf16_round(rng.standard_normal(T * hs).astype(np.float32))
    hf = dev.put(fill, True)
    for h_ in (hq, hk, hv):
        for i in range(B * H):
            dev.cuda.copy(T * hs, hf, h_, 0, i * T * hs)
    data = {}
    for (b, h) in picks:
        q, k, v = (bf16_round(rng.standard_normal((T, hs)).astype(np.float32)) for _ in range(3))
        data[(b, h)] = (q, k, v)
        for arr, hd in ((q, hq), (k, hk), (v, hv)):
            ht = dev.put(arr, True)
            dev.cuda.copy(T * hs, ht, hd, 0, (b * H + h) * T * hs)
    hm = dev.put(np.tril(np.ones((T, T), np.float32)))
    hc, ha = dev.cuda.CreateCuDNN(), dev.cuda.CreateAttn()
    dev.cuda.SetAttn(hc, ha, 0, False, B, T, H, hs, 0.0)
    dev.cuda.AttnScaledDotProductForward(hc, ha, T, hq, hk, hv, hm, hy, False)
    y = dev.get(hy, (B, H, T, hs))
    dev.cuda.FreeAttn(ha)
    dev.cuda.FreeCuDNN(hc)
    assert np.all(np.isfinite(y))
    tri = np.tril(np.ones((T, T), bool))
    for (b, h), (q, k, v) in data.items():
        s_ = (q.astype(np.float64) @ k.astype(np.float64).T) / np.sqrt(hs)
        s_ = np.where(tri, s_, -np.inf)
        p = np.exp(s_ - s_.max(-1, keepdims=True))
        ref = (p / p.sum(-1, keepdims=True)) @ v.astype(np.float64)
        assert_close(y[b, h], ref, BF16_RTOL, "long-context causal attention, head (%d, %d)" % (b, h))
    # every other head holds the same q = k = v block: identical outputs, and row 0 attends to key 0 only
    same = [(b, h) for b in range(B) for h in range(H) if (b, h) not in data]
    assert_close(y[same[0]][0], fill.reshape(T, hs)[0], BF16_RTOL, "row 0 returns V[0]")
    for bh in same[1:]:
        assert np.array_equal(y[bh], y[same[0]]), "heads with identical inputs differ: %s" % (bh,)


# ---- decode attention, 32 heads x 128, cache 4096 --------------------------------------------

def _decode_row_ref(q, k, v):
    """fp64 closed form of one (batch, head) row: softmax(k q / sqrt(hs)) v."""
    s = (k.astype(np.float64) @ q.astype(np.float64)) / np.sqrt(float(q.shape[-1]))
    p = np.exp(s - s.max())
    p /= p.sum()
    return p @ v.astype(np.float64)


@pytest.mark.parametrize("B", [1, 32])
def test_attn_decode_7b_head_shape_L4096(dev, B):
    H, L, hs = 32, 4096, 128
    rng = np.random.default_rng(4096 + B)
    q = rng.standard_normal((B, H, hs), dtype=np.float32)
    k = rng.standard_normal((B, H, L, hs), dtype=np.float32)
    v = rng.standard_normal((B, H, L, hs), dtype=np.float32)
    rows = [(int(b), int(h)) for b, h in zip(rng.integers(0, B, 12), rng.integers(0, H, 12))] + [(0, 0), (B - 1, H - 1)]
    for half in (False, True):
        print("decode attention B=%d L=%d %s" % (B, L, "bf16" if half else "fp32"), flush=True)
        hq, hk, hv, hy = dev.put(q, half), dev.put(k, half), dev.put(v, half), dev.zeros(q.size, half)
        dev.cuda.AttnDecodeForward(B, H, H, hs, L, hq, hk, hv, hy, H * L * hs, L * hs, hs)
        y = dev.get(hy, q.shape)
        assert np.all(np.isfinite(y))
        rnd = bf16_round if half else (lambda a: a)
        for (b, h) in rows:
            # a seeded sample of rows in fp64 (the whole cache in fp64 would be 17 GB at batch 32)
            ref = _decode_row_ref(rnd(q[b, h]), rnd(k[b, h]), rnd(v[b, h]))
            assert_close(y[b, h], ref, BF16_RTOL if half else FP32_RTOL, "row (%d,%d)" % (b, h))
        for hnd in (hq, hk, hv, hy):
            dev.cuda.FreeMemory(hnd)
            dev.handles.remove(hnd)


@pytest.mark.parametrize("half", [False, True])
def test_attn_decode_7b_head_shape_with_rope_and_append_B32_L4096(dev, half):
    # the form the microbenchmark times: rotate q and the newest key at position L - 1 (theta 10000), append key and
    # value to the caches, then attend over all L positions
    B, H, L, hs = 32, 32, 4096, 128
    rng = np.random.default_rng(77)
    q = rng.standard_normal((B, H, hs), dtype=np.float32)
    kn = rng.standard_normal((B, H, hs), dtype=np.float32)
    vn = rng.standard_normal((B, H, hs), dtype=np.float32)
    k = rng.standard_normal((B, H, L, hs), dtype=np.float32)
    v = rng.standard_normal((B, H, L, hs), dtype=np.float32)
    hr = dev.cuda.CreateRope(0, 0, B * H * hs, B, L, H, hs, 10000.0)
    hq, hkn, hvn, hk, hv, hy = (dev.put(a, half) for a in (q, kn, vn, k, v, np.zeros_like(q)))
    dev.cuda.AttnDecodeForward(B, H, H, hs, L, hq, hk, hv, hy, H * L * hs, L * hs, hs, 0.0, hr, hkn, hvn)
    y = dev.get(hy, q.shape)
    cos, sin = R.rope_tables(L, hs)
    rnd = bf16_round if half else (lambda a: a)

    def rot(x):
        x = rnd(x).astype(np.float64)
        o = x.copy()
        o[..., 0::2] = x[..., 0::2] * cos[L - 1] - x[..., 1::2] * sin[L - 1]
        o[..., 1::2] = x[..., 0::2] * sin[L - 1] + x[..., 1::2] * cos[L - 1]
        return o

    rq, rk = rnd(rot(q).astype(np.float32)), rnd(rot(kn).astype(np.float32))   # stored back in the storage type
    tol = BF16_RTOL if half else FP32_RTOL
    for b, h in [(0, 0), (31, 31), (7, 19), (20, 3), (13, 13), (29, 8)]:
        kk, vv = rnd(k[b, h]).astype(np.float64), rnd(v[b, h]).astype(np.float64)
        kk[L - 1], vv[L - 1] = rk[b, h], rnd(vn[b, h])
        assert_close(y[b, h], _decode_row_ref(rq[b, h], kk, vv), tol, "row (%d,%d)" % (b, h))
    # the caches hold the appended rows
    kc = dev.get(hk, k.shape)
    # the rotation factors at position 4095 come from fp32 angles of up to 4095 radians (rope.cu:544-553): one unit in
    # the last place of a frequency (powf of the C library against numpy's) moves such an angle by 2.4e-4, and the
    # rotated key with it.  The bound is that, not fp32 round-off; the attention output above is held to the parity bar.
    assert_close(kc[:, :, L - 1], rk, tol if half else 4e-4, "appended key rows")
    assert np.array_equal(kc[:, :, L - 2], rnd(k[:, :, L - 2]))
    assert np.array_equal(dev.get(hv, v.shape)[:, :, L - 1], rnd(vn))


# ---- encoder-decoder attention, d_model 512, 8 x 64, batch 32, 256 / 128, bf16 ----------------

def test_encdec_attention_config_bf16(dev):
    rng = np.random.default_rng(7)
    B, Ts, Tt, C, H = 32, 256, 128, 512, 8
    slen, tlen = rng.integers(32, Ts + 1, B), rng.integers(16, Tt + 1, B)
    W = {k: bf16_round((rng.standard_normal((C, C)) * 0.02).astype(np.float32)) for k in ("wq", "wk", "wv", "wo")}
    W.update({k: np.zeros(C, np.float32) for k in ("bq", "bk", "bv", "bo")})
    src = bf16_round(rng.standard_normal((B, Ts, C)).astype(np.float32))
    tgt = bf16_round(rng.standard_normal((B, Tt, C)).astype(np.float32))
    enc_mask = (np.arange(Ts)[None, :] < slen[:, None]).astype(np.float32)
    dec_mask = ((np.arange(Tt)[None, :] < tlen[:, None])[:, None, :] * np.tril(np.ones((Tt, Tt)))[None]).astype(np.float32)
    bs, bt, top = Blob(dev.cuda, src.shape, half=True), Blob(dev.cuda, tgt.shape, half=True), Blob(dev.cuda, half=True)
    bs.mutable_cpu_data, bt.mutable_cpu_data = src, tgt
    bm, bdm = Blob(dev.cuda, (B, Ts, 1, 1)), Blob(dev.cuda, (B, Tt, Tt, 1))
    bm.mutable_cpu_data, bdm.mutable_cpu_data = enc_mask, dec_mask
    args = (W["wq"], W["bq"], W["wk"], W["bk"], W["wv"], W["bv"], W["wo"], W["bo"], H)

    print("encoder self attention, key-padding mask, bf16", flush=True)
    enc = MultiheadAttentionLayer(dev.cuda, H, C, Ts, True, True, half=True)
    enc.Setup(bs, bs, bs, W)
    enc.Forward(bs, bs, bs, bm, top)
    ref = R.multihead_attention(src, src, src, *args, enc_mask, "key", dtype=np.float64)["y"]
    # rows of padded queries are defined too (their keys are masked the same way); compare everything
    assert_close(top.mutable_cpu_data, ref, BF16_RTOL, "encoder self attention bf16")

    print("decoder self attention, per-sequence causal-and-padding mask, bf16", flush=True)
    ref = R.multihead_attention(tgt, tgt, tgt, *args, dec_mask, "full", dtype=np.float64)["y"]
    # 16-bit storage goes through the fused handle only: the explicit chain's batched MatMul (gemm2) refuses
    # half-size memory, as the reference's does (math.cu:1777-1778)
    dec = MultiheadAttentionLayer(dev.cuda, H, C, Tt, True, True, half=True, fuse_batch_qk_mask=True)
    dec.Setup(bt, bt, bt, W)
    dec.Forward(bt, bt, bt, bdm, top)
    assert_close(top.mutable_cpu_data, ref, BF16_RTOL, "decoder self attention bf16")

    print("cross attention T_q 128 / T_k 256, source key-padding mask, bf16", flush=True)
    cross = MultiheadAttentionLayer(dev.cuda, H, C, Ts, True, True, half=True)
    cross.Setup(bt, bs, bs, W)
    cross.Forward(bt, bs, bs, bm, top)
    ref = R.multihead_attention(tgt, src, src, *args, enc_mask, "key", dtype=np.float64)["y"]
    assert_close(top.mutable_cpu_data, ref, BF16_RTOL, "cross attention bf16")


# ---- causal self attention layer, B = 8, T = 1024, C = 768 ------------------------------------

@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("N", [2304, 768, 1536])
def test_inner_product_gemm_at_layer_shapes(dev, half, N):
    # InnerProductLayer.forward: gemm(false, true, M, N, K, 1, X, W, 0, Y), W stored [N, K]
    M, K = 8192, 768
    rng = np.random.default_rng(N)
    x = bf16_round(rng.standard_normal((M, K), dtype=np.float32))
    w = bf16_round((rng.standard_normal((N, K), dtype=np.float32) * 0.02))
    hx, hw, hy = dev.put(x, half), dev.put(w, half), dev.zeros(M * N, half)
    dev.cuda.gemm(False, True, M, N, K, 1.0, hx, hw, 0.0, hy)
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    assert_close(dev.get(hy, (M, N)), ref, BF16_RTOL if half else FP32_RTOL, "gemm %dx%dx%d" % (M, N, K))
    # every tile of the walk was written: no row or column band left at zero
    y = dev.get(hy, (M, N))
    assert np.count_nonzero(np.abs(y).max(axis=1) == 0) == 0 and np.count_nonzero(np.abs(y).max(axis=0) == 0) == 0


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("H,hs", [(12, 64), (8, 64)])
def test_qkv_proj_heads_at_layer_shapes(dev, half, H, hs):
    # the fused QKV projection over 8 x 1024 tokens: in 16-bit storage 8192 x 2304 x 768 is 256 tiles of 256 x 288 and
    # 8192 x 1536 x 512 is 256 tiles of 256 x 192 (one workgroup per CU each); every element of q, k, v against the checker
    B, T, C = 8, 1024, H * hs
    rng = np.random.default_rng(C)
    x = bf16_round(rng.standard_normal((B, T, C), dtype=np.float32))
    w = bf16_round(rng.standard_normal((3 * C, C), dtype=np.float32) * 0.02)
    bv = bf16_round(rng.standard_normal(3 * C, dtype=np.float32) * 0.1)
    hx, hw, hb = dev.put(x, half), dev.put(w, half), dev.put(bv, half)
    hq, hk, hv = (dev.zeros(B * T * C, half) for _ in range(3))
    dev.cuda.QkvProjHeads(B, T, H, hs, hx, hw, hb, hq, hk, hv)
    ref = R.inner_product(x, w, bv, np.float64).reshape(B, T, 3, H, hs).transpose(2, 0, 3, 1, 4)
    for i, (name, h) in enumerate(zip("qkv", (hq, hk, hv))):
        assert_close(dev.get(h, (B, H, T, hs)), ref[i], BF16_RTOL if half else FP32_RTOL, name)
    # the same with the rotation of q and k in the epilogue (the wide tiles' store path in 16-bit storage)
    hr = dev.cuda.CreateRope(0, 0, B * T * C, B, T, H, hs, 10000.0)
    dev.cuda.QkvProjHeads(B, T, H, hs, hx, hw, hb, hq, hk, hv, hr)
    dev.cuda.FreeRope(hr)
    qkv = ref.transpose(1, 3, 0, 2, 4)      # (B, T, 3, H, hs)
    for i, (name, h) in enumerate(zip("qkv", (hq, hk, hv))):
        want = R.rope_forward(qkv[:, :, i], T, H, hs, dtype=np.float64).reshape(B, T, H, hs) if i < 2 else qkv[:, :, i]
        assert_close(dev.get(h, (B, H, T, hs)), want.transpose(0, 2, 1, 3), BF16_RTOL if half else FP32_RTOL, name + " rotated")


@pytest.mark.parametrize("half", [False, True])
def test_causal_self_attention_layer_B8_T1024_C768(dev, half):
    B, T, C, H = 8, 1024, 768, 12
    rng = np.random.default_rng(0)
    x = bf16_round(rng.standard_normal((B, T, C), dtype=np.float32))
    w_attn = bf16_round(rng.standard_normal((3 * C, C), dtype=np.float32) * 0.02)
    w_proj = bf16_round(rng.standard_normal((C, C), dtype=np.float32) * 0.02)
    b_attn, b_proj = np.zeros(3 * C, np.float32), np.zeros(C, np.float32)
    layer = CausalSelfAttentionLayer(dev.cuda, H, C, T, True, True, half=half)
    bottom, top = Blob(dev.cuda, x.shape, half=half), Blob(dev.cuda, half=half)
    bottom.mutable_cpu_data = x
    layer.Setup(bottom, w_attn, b_attn, w_proj, b_proj)
    layer.Forward(bottom, top)
    y = top.mutable_cpu_data
    # the checker one sequence at a time (the (H, T, T) scores of one sequence in fp64 are 100 MB)
    for b in range(B):
        ref = R.causal_self_attention(x[b:b + 1], w_attn, b_attn, w_proj, b_proj, H, dtype=np.float64)["y"]
        assert_close(y[b:b + 1], ref, BF16_RTOL if half else FP32_RTOL, "layer output, sequence %d" % b)
