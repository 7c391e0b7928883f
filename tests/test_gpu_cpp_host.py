"""Runs the C++ host-side parity program (tests/cpp/host_parity.cpp): the libraries driven from C++ through
include/mycaffe_hip_host.hpp, as the reference's C# host drives its DLL through CudaControl."""
import os
import subprocess

import numpy as np
import pytest

from mycaffe_amd import build as B
from mycaffe_amd.cudadnn import default_library_path, llama2_extension_path
from tests.conftest import GOLDEN

pytestmark = pytest.mark.gpu


def _program():
    path = os.path.normpath(B.host_program_path())
    if not os.path.exists(path):
        B.build_host_program(verbose=False)
    return path


def test_cpp_host_parity_program(tmp_path):
    from oracle import llama2 as O
    cfg = dict(dim=64, hidden_dim=172, n_layers=2, n_heads=4, n_kv_heads=4, vocab_size=97, seq_len=48)
    blob, _ = O.random_weights(cfg, seed=11, shared_classifier=False, std=0.3)
    ckpt = str(tmp_path / "tiny.bin")
    O.write_checkpoint_v1(ckpt, cfg, blob, False)
    prompt = [5, 17, 3, 90]
    n_steps = 40
    r = subprocess.run([_program(), default_library_path(), GOLDEN, llama2_extension_path(), ckpt, str(n_steps)] + [str(p) for p in prompt],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    print(r.stdout)
    assert r.returncode == 0, r.stdout
    lines = r.stdout.splitlines()
    assert sum(l.startswith("PASS") for l in lines) == 19 and not any(l.startswith("FAIL") for l in lines)
    ids = [int(t) for t in next(l for l in lines if l.startswith("IDS")).split()[1:]]
    ref = O.Llama(cfg, blob, False).generate_greedy(np.array(prompt), n_steps)
    assert ids == list(ref)
