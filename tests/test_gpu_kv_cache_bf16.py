"""GPU parity of the engine's 16-bit KV cache (SET_OPTION 8): keys (after rotation) and values are rounded to bfloat16
when they enter the cache, and the step that appends them attends over the rounded row too.  The CPU checker has the
same rounding as a checker-only option (pinned in tests/test_oracle_llama.py), so logits are compared position by
position; activations and weights stay fp32 here."""
import numpy as np
import pytest

from mycaffe_amd.cudadnn import CudaDnn
from mycaffe_amd.llm_inference import LlmInference
from oracle import llama2 as O
from tests.conftest import FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu

# The two sides compute the fp32 key / value with different summation orders; where they differ in the last bit next to
# a rounding boundary the cached bfloat16 differs by one step (0.4 % of that element).  A few such elements per
# generation move the logits by some 1e-4 of their maximum, so the comparison allows 1e-3: ten times tighter than the
# 1e-2 bar of 16-bit storage, and far below the effect of the rounding itself (checked below).
KV_RTOL = 1e-3

TINY = dict(dim=64, hidden_dim=172, n_layers=3, n_heads=4, n_kv_heads=4, vocab_size=512, seq_len=64)
HS64 = dict(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=512, seq_len=256)
C1 = dict(dim=288, hidden_dim=768, n_layers=6, n_heads=6, n_kv_heads=6, vocab_size=32000, seq_len=256)


@pytest.fixture()
def llm():
    cuda = CudaDnn(0)
    inf = LlmInference(cuda)
    inf.Initialize(fTemperature=0.0)
    yield inf
    inf.CleanUp()
    cuda.Dispose()


def _cpu(cfg, blob, prompt, n, rounded):
    O.set_kv_bf16(rounded)
    try:
        return O.Llama(cfg, blob).generate_greedy(prompt, n, want_logits=True)
    finally:
        O.set_kv_bf16(False)


def _first_max(logits):
    return np.argmax(logits, axis=-1)   # numpy returns the first of equal maxima


def _compare(ids, logits, ref_ids, ref_logits, tol, what):
    """ids are the first-max argmax of the device logits; they equal the checker's up to the first position where the
    checker's top-2 gap is within the tolerance; logits agree up to and including that position."""
    assert np.array_equal(ids, _first_max(logits)), what + ": id is not the first-max argmax of the device logits"
    same = np.array_equal(ids, ref_ids)
    upto = len(ids) if same else int(np.argmax(np.asarray(ids) != np.asarray(ref_ids))) + 1
    assert_close(logits[:upto], ref_logits[:upto], tol, what + " logits")
    if not same:
        top2 = np.sort(ref_logits[upto - 1])[-2:]
        gap = (top2[1] - top2[0]) / max(float(np.abs(ref_logits[upto - 1]).max()), 1e-30)
        assert gap < tol, "%s: ids differ at step %d where the checker's top-2 gap is %.3e" % (what, upto - 1, gap)
    return same


@pytest.mark.parametrize("name,cfg,std,nP,n", [("tiny", TINY, 0.2, 9, 40), ("gqa", dict(TINY, n_kv_heads=2), 0.2, 17, 48),
                                               ("hs64", HS64, 0.08, 100, 160), ("c1", C1, 0.02, 8, 64)])
def test_bf16_cache_logits_and_ids(llm, tmp_path, name, cfg, std, nP, n):
    blob, _ = O.random_weights(cfg, seed=33, shared_classifier=False, std=std)
    path = str(tmp_path / (name + ".bin"))
    O.write_checkpoint_v1(path, cfg, blob, False)
    llm.Load(path)
    prompt = np.random.default_rng(8).integers(3, cfg["vocab_size"], nP)
    ref_ids, ref_logits = _cpu(cfg, blob, prompt, n, True)
    plain_ids, plain_logits = _cpu(cfg, blob, prompt, n, False)
    effect = np.abs(ref_logits - plain_logits).max() / np.abs(plain_logits).max()
    assert effect > KV_RTOL, "the rounding is not visible in this case (%.2e): the test would prove nothing" % effect
    llm.SetOption(8, 1)
    for batched_prompt in (0, 1):
        llm.SetOption(7, batched_prompt)
        ids, logits = llm.GenerateIds(prompt, n, want_logits=True)        # eager launches
        assert llm.LastPrefill()[1] == (nP if batched_prompt else 0)
        _compare(ids, logits, ref_ids, ref_logits, KV_RTOL, "%s, 16-bit cache, batched prompt pass %d" % (name, batched_prompt))
        assert np.array_equal(llm.GenerateIds(prompt, n), ids)            # graph replays
        assert llm.LastRunUsedGraph()
    # back to the fp32 cache: the run state is rebuilt and the plain checker is matched at the fp32 bar again
    llm.SetOption(8, 0)
    ids, logits = llm.GenerateIds(prompt, n, want_logits=True)
    _compare(ids, logits, plain_ids, plain_logits, FP32_RTOL, name + ", fp32 cache again")


def test_bf16_cache_batch_with_multi_iteration_splits(llm, tmp_path):
    """40 sequences x 4 heads of size 64 over a 512-position cache: the fused decode attention takes two splits of 256
    rows per (sequence, head), i.e. several iterations of cache rows per split, and appends the new key / value through the
    cache (the path batch 1 does not take).  Every row against its own CPU run with the rounding option.  This model is
    a sensitive one (the rounding itself moves its logits by more than their maximum over 160 steps), so one-step
    differences of cached elements grow over the 200 positions: 3e-3 here, still well inside the 16-bit bar of 1e-2."""
    cfg = dict(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=512, seq_len=512)
    blob, _ = O.random_weights(cfg, seed=12, shared_classifier=False, std=0.08)
    path = str(tmp_path / "gqa_batch.bin")
    O.write_checkpoint_v1(path, cfg, blob, False)
    llm.Load(path)
    llm.SetOption(8, 1)
    B, nP, n = 40, 6, 200
    prompts = np.random.default_rng(3).integers(3, cfg["vocab_size"], (B, nP))
    ids, logits = llm.GenerateBatch(prompts, n, want_logits=True)
    parted = 0
    for b in range(B):
        ref_ids, ref_logits = _cpu(cfg, blob, prompts[b], n, True)
        parted += 0 if _compare(ids[b], logits[b], ref_ids, ref_logits, 3 * KV_RTOL, "sequence %d" % b) else 1
    assert parted <= 4, "%d of %d sequences parted from the checker" % (parted, B)


def test_bf16_cache_is_refused_quietly_for_head_sizes_it_cannot_pack(llm, tmp_path):
    """A 16-byte chunk of a bfloat16 cache row holds 8 dims of one head: with a head size that is not a multiple of 8 the
    option leaves the cache in fp32 and results stay those of the plain checker."""
    cfg = dict(dim=48, hidden_dim=128, n_layers=2, n_heads=4, n_kv_heads=4, vocab_size=300, seq_len=48)   # head size 12
    blob, _ = O.random_weights(cfg, seed=2, shared_classifier=False, std=0.2)
    path = str(tmp_path / "hs12.bin")
    O.write_checkpoint_v1(path, cfg, blob, False)
    llm.Load(path)
    llm.SetOption(8, 1)
    prompt = np.array([5, 9, 200, 17])
    ids, logits = llm.GenerateIds(prompt, 30, want_logits=True)
    ref_ids, ref_logits = _cpu(cfg, blob, prompt, 30, False)
    _compare(ids, logits, ref_ids, ref_logits, FP32_RTOL, "head size 12")
