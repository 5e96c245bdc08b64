"""A host in plain C (tests/c_host/shim_twin.c): the Rust shim's call sequence compiled with gcc
against include/coeus.h and linked to the shared library, no Python and no ctypes in the process
that makes the calls.  The CPU part runs the entry points that need no device; the GPU part builds
the reference's default-initialised model and compares forward()'s logits with the Python host's
and the oracle's."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBDIR = os.path.join(ROOT, "coeus_amd")


@pytest.fixture(scope="module")
def twin(tmp_path_factory):
    exe = tmp_path_factory.mktemp("c_host") / "shim_twin"
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Werror", "-O1", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "c_host", "shim_twin.c"), "-o", str(exe),
                           "-L", LIBDIR, "-l:libcoeus_mi355x.so", f"-Wl,-rpath,{LIBDIR}"])
    return str(exe)


def test_c_host_without_a_device(twin, tmp_path):
    r = subprocess.run([twin, "host", str(tmp_path / "m.rustllm")], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "host ok" in r.stdout


@pytest.mark.gpu
def test_c_host_forward_equals_python_host_and_oracle(twin, tmp_path, orc):
    from coeus_amd import Transformer250MConfig, TransformerModelPlugin

    ids = [100, 200, 30, 7, 299]
    out = tmp_path / "logits.f32"
    r = subprocess.run([twin, "forward", str(out)] + [str(i) for i in ids], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(out, dtype=np.float32)
    kw = dict(hidden_dim=64, num_layers=2, num_heads=4, intermediate_dim=128, vocab_size=300, max_seq_len=32)
    py = TransformerModelPlugin().create_builder().build(Transformer250MConfig(**kw)).forward(ids)
    assert np.array_equal(got, py)  # the same library, the same kernels, another host language
    oc = orc.config_from_kwargs(kw)
    rc, want = orc.forward(oc, orc.init_default(orc.num_parameters(oc), 64), ids)
    assert rc == 0 and np.abs(got - want).max() / np.abs(want).max() < 1e-3
    r = subprocess.run([twin, "errors"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "errors ok" in r.stdout, r.stdout + r.stderr
