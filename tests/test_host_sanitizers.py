"""The host logic of the library (errors, configuration and parameter layout, the .rustllm reader and
writer with their error cases, the byte-pair tokenizer) built with AddressSanitizer and
UndefinedBehaviorSanitizer on the host pass and run through its own tests in a child process.
Device code is not sanitized and not part of this build."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_sources_clean_under_asan_and_ubsan():
    from coeus_amd.build import asan_runtime, build_host_sanitized

    rt = asan_runtime()
    if rt is None:
        pytest.skip("the compiler ships no shared AddressSanitizer runtime")
    lib = build_host_sanitized()
    env = dict(os.environ)
    env.update(LD_PRELOAD=rt, COEUS_HOST_LIB=lib,
               ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0:abort_on_error=0:exitcode=99",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1:exitcode=98")
    r = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "not gpu", "-p", "no:cacheprovider",
                        "tests/test_rustllm_file.py", "tests/test_tokenizer.py",
                        "tests/test_host_cpu.py::test_config_defaults_validate_and_counts",
                        "tests/test_host_cpu.py::test_default_init_and_positional_table_match_oracle_bitwise",
                        "tests/test_abi_layout.py::test_last_error_is_thread_local"],
                       cwd=ROOT, env=env, capture_output=True, text=True, timeout=600)
    out = r.stdout + r.stderr
    assert "AddressSanitizer" not in out and "runtime error:" not in out, out[-4000:]
    assert r.returncode == 0, out[-4000:]
    assert " passed" in out
