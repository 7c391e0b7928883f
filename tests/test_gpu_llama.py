"""GPU parity of the llama2 extension (loaded through CREATE_EXTENSION, driven by the
LlmInference mirror) against the CPU checker: logits of every step and greedy ids."""
import os

import numpy as np
import pytest

from mycaffe_amd.cudadnn import CudaDnn, CudaDnnError
from mycaffe_amd.llm_inference import LlmInference
from oracle import llama2 as O
from tests.conftest import BF16_RTOL, FP32_RTOL, assert_close, bf16_round

pytestmark = pytest.mark.gpu

TINY = dict(dim=64, hidden_dim=172, n_layers=3, n_heads=4, n_kv_heads=4, vocab_size=512, seq_len=64)
C1 = dict(dim=288, hidden_dim=768, n_layers=6, n_heads=6, n_kv_heads=6, vocab_size=32000, seq_len=256)


@pytest.fixture()
def llm():
    cuda = CudaDnn(0)
    inf = LlmInference(cuda)
    inf.Initialize(fTemperature=0.0)
    yield inf
    inf.CleanUp()
    cuda.Dispose()


def _margin(logits):
    s = np.sort(logits, axis=-1)
    return (s[:, -1] - s[:, -2]) / np.abs(s[:, -1]).clip(1e-30)


def _check_ids(ids, ref_ids, ref_logits, what):
    """Bit-exact ids; a mismatch is only tolerated (and reported) where the checker's own
    top-2 logit gap is below the fp32 parity tolerance, i.e. the argmax is undetermined."""
    if np.array_equal(ids, ref_ids):
        return
    first = int(np.argmax(ids != ref_ids))
    m = _margin(ref_logits[first:first + 1])[0]
    assert m < FP32_RTOL, "%s: ids differ at step %d with a decisive margin %.3e" % (what, first, m)
    pytest.skip("%s: near-tie (relative top-2 gap %.2e) at step %d; ids before it are identical" % (what, m, first))


@pytest.mark.parametrize("cfg,shared,std", [(TINY, False, 0.2), (TINY, True, 0.2), (dict(TINY, n_kv_heads=2), False, 0.2)])
def test_logits_and_ids_tiny(llm, tmp_path, cfg, shared, std):
    blob, views = O.random_weights(cfg, seed=7, shared_classifier=shared, std=std)
    rng = np.random.default_rng(1)
    for k in ("rms_att", "rms_ffn", "rms_final"):
        views[k][...] = 1 + 0.2 * rng.standard_normal(views[k].shape).astype(np.float32)
    path = str(tmp_path / "tiny.bin")
    O.write_checkpoint_v1(path, cfg, blob, shared)
    llm.Load(path)
    assert llm.QueryStatus() == (1.0, 1)
    prompt = rng.integers(3, cfg["vocab_size"], 8)
    n = 48
    ids, logits = llm.GenerateIds(prompt, n, want_logits=True)
    ref_ids, ref_logits = O.Llama(cfg, blob, shared).generate_greedy(prompt, n, want_logits=True)
    assert_close(logits, ref_logits, FP32_RTOL, "logits")
    _check_ids(ids, ref_ids, ref_logits, "tiny")
    # the captured-graph path (no logits requested) gives the same ids as the eager one
    ids2 = llm.GenerateIds(prompt, n)
    assert np.array_equal(ids2, ids)
    llm.SetOption(3, 0)
    assert np.array_equal(llm.GenerateIds(prompt, n), ids)


def test_reference_cpu_config_greedy_256_tokens(llm, tmp_path):
    """dim 288 / 6 layers / 6 heads x 48 / ffn 768 / vocab 32000 / seq 256, N(0, 0.02) weights,
    RMSNorm weights 1, unshared classifier; 8 seeded prompt ids, greedy to 256 tokens."""
    blob, _ = O.random_weights(C1, seed=1234, shared_classifier=False, std=0.02)
    path = str(tmp_path / "c1.bin")
    O.write_checkpoint_v1(path, C1, blob, False)
    llm.Load(path)
    prompt = np.random.default_rng(1).integers(3, 32000, 8)
    ids = llm.GenerateIds(prompt, 256)
    ref_ids, ref_logits = O.Llama(C1, blob).generate_greedy(prompt, 256, want_logits=True)
    _check_ids(ids, ref_ids, ref_logits, "C1")
    ms, steps = llm.QueryTiming()
    assert steps == 248 and ms > 0


def test_bf16_weight_storage(llm, tmp_path):
    blob, _ = O.random_weights(TINY, seed=9, std=0.2)
    path = str(tmp_path / "tiny.bin")
    O.write_checkpoint_v1(path, TINY, blob, False)
    llm.SetOption(1, 1)
    llm.Load(path)
    prompt = np.arange(5, 13)
    ids, logits = llm.GenerateIds(prompt, 40, want_logits=True)
    # same arithmetic on bf16-rounded weights: isolates the storage rounding
    rb = bf16_round(blob)
    ref_ids, ref_logits = O.Llama(TINY, rb).generate_greedy(prompt, 40, want_logits=True)
    assert_close(logits, ref_logits, FP32_RTOL, "bf16-weight logits vs checker on rounded weights")
    _check_ids(ids, ref_ids, ref_logits, "bf16 weights")
    # and within the 16-bit tolerance of the fp32 model
    _, full = O.Llama(TINY, blob).generate_greedy(prompt, 1, want_logits=True)
    assert_close(logits[:1], full, BF16_RTOL, "bf16 vs fp32 model")


def test_batch_generation_matches_independent_sequences(llm, tmp_path):
    blob, _ = O.random_weights(TINY, seed=11, std=0.2)
    path = str(tmp_path / "tiny.bin")
    O.write_checkpoint_v1(path, TINY, blob, False)
    llm.Load(path)
    prompts = np.random.default_rng(2).integers(3, TINY["vocab_size"], (5, 6))
    out = llm.GenerateBatch(prompts, 40)
    for b in range(5):
        ref_ids, ref_logits = O.Llama(TINY, blob).generate_greedy(prompts[b], 40, want_logits=True)
        _check_ids(out[b], ref_ids, ref_logits, "batch row %d" % b)


def test_error_paths(llm, tmp_path):
    with pytest.raises(CudaDnnError) as e:
        llm.Load(str(tmp_path / "missing.bin"))
    assert e.value.code == 10002
    blob, _ = O.random_weights(TINY, seed=1)
    path = str(tmp_path / "t.bin")
    O.write_checkpoint_v1(path, TINY, blob, False)
    with pytest.raises(CudaDnnError) as e:
        llm.Load(path, str(tmp_path / "no_tokenizer.bin"))
    assert e.value.code == 10003
    with pytest.raises(CudaDnnError) as e:   # generate before load
        llm.GenerateIds([1, 2, 3], 8)
    assert e.value.code == 10004
    bad = tmp_path / "bad.bin"
    bad.write_bytes(b"\0" * 300)
    with pytest.raises(CudaDnnError) as e:
        llm.Load(str(bad))
    assert e.value.code == 10001
    llm.Load(path)
    with pytest.raises(CudaDnnError):        # token id outside the vocabulary
        llm.GenerateIds([TINY["vocab_size"] + 5], 4)
    text, end = llm.QueryResponse()
    assert text == "" and not end or end
    llm.CancelGenerate()
