"""CPU-only checks of the product's host side: the C-ABI library loads, exports every symbol
include/coeus.h declares, and its host logic (config, layout, init, positional table, error
mapping) agrees with the oracle.  No kernel is launched here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from coeus_amd import (ConfigError, DeviceError, Transformer250MConfig, TransformerModelBuilder,
                       TransformerModelPlugin, _lib)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "coeus.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(coeus_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 40
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/coeus.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names  # and nothing is bound that the header does not declare


def test_config_defaults_validate_and_counts(orc):
    lib = _lib.load()
    c = _lib.CConfig()
    lib.coeus_config_default(C.byref(c))
    oc = orc.default_config()
    for f, _ in _lib.CConfig._fields_:
        assert getattr(c, f) == getattr(oc, f), f
    cfg = Transformer250MConfig()
    cfg.validate()
    assert cfg.num_parameters() == 163_087_441 == orc.num_parameters(oc)  # MT:541-580
    assert cfg.used_parameters() == 162_250_752
    # the invalid cases of CM:792-806, with the reference's messages
    with pytest.raises(ConfigError, match="must be divisible by number of heads"):
        Transformer250MConfig(hidden_dim=767).validate()
    with pytest.raises(ConfigError, match="Number of layers must be greater than 0"):
        Transformer250MConfig(num_layers=0).validate()
    with pytest.raises(ConfigError, match="Vocabulary size must be greater than 0"):
        Transformer250MConfig(vocab_size=0).validate()
    with pytest.raises(ConfigError, match="Maximum sequence length must be greater than 0"):
        Transformer250MConfig(max_seq_len=0).validate()
    with pytest.raises(ConfigError):
        Transformer250MConfig(num_heads=0).validate()  # a division by zero in the reference
    with pytest.raises(ConfigError):
        Transformer250MConfig(weight_dtype="q4_0", hidden_dim=48, num_heads=4).validate()
    with pytest.raises(ConfigError):
        Transformer250MConfig(activation="relu").validate()
    # parameter counts for extension shapes agree with the oracle's layout
    for kw in (dict(hidden_dim=64, num_layers=3, num_heads=4, head_dim=8, intermediate_dim=96,
                    vocab_size=100, max_seq_len=16, use_bias=False, activation="silu_gated"),
               dict(hidden_dim=4096, num_layers=32, num_heads=32, intermediate_dim=11008,
                    vocab_size=32000, max_seq_len=4096, use_bias=False, activation="silu_gated")):
        cfg = Transformer250MConfig(**kw)
        oc = orc.config_from_kwargs(kw)
        assert cfg.num_parameters() == orc.num_parameters(oc)
        assert cfg.used_parameters() == orc.layout(oc).used_params


def test_default_init_and_positional_table_match_oracle_bitwise(orc):
    lib = _lib.load()
    n = 300_000
    p = np.empty(n, dtype=np.float32)
    assert lib.coeus_init_default_parameters(p.ctypes.data, n, 768) == 0
    assert np.array_equal(p.view(np.uint32), orc.init_default(n, 768).view(np.uint32))
    t = np.empty((64, 48), dtype=np.float32)
    assert lib.coeus_positional_encoding(64, 48, t.ctypes.data) == 0
    assert np.array_equal(t.view(np.uint32), orc.positional_encoding(64, 48).view(np.uint32))


def test_plugin_surface_without_a_device():
    p = TransformerModelPlugin()
    assert p.id() == "transformer_model" and p.version() == (0, 1, 0)  # MT:1127-1134
    b = p.create_builder()
    assert isinstance(b, TransformerModelBuilder)
    with pytest.raises(ConfigError):
        b.build(Transformer250MConfig(hidden_dim=767))  # validation comes first (MT:590)
    lib = _lib.load()
    name = C.create_string_buffer(64)
    if lib.coeus_device_info(name, 64, None, None) != 0:
        # no GPU in this container: building a model must fail loudly, never fall back
        small = Transformer250MConfig(hidden_dim=32, num_layers=1, num_heads=2, intermediate_dim=32,
                                      vocab_size=16, max_seq_len=8)
        with pytest.raises(DeviceError, match="no HIP device"):
            b.build(small)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "coeus_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"


def test_profiler_detection_reads_the_environment():
    """coeus_profiler_attached: 0 in a plain process, 1 when a tool library is named the way a
    profiler's launcher names it (HSA_TOOLS_LIB is read as text here: without a GPU nothing loads
    it).  Looked up once per process, so each case is a process of its own."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = "from coeus_amd import _lib; print(_lib.load().coeus_profiler_attached())"
    for extra, want in [({}, "0"), ({"HSA_TOOLS_LIB": "libroctracer64.so"}, "1"),
                        ({"HSA_TOOLS_LIB": "librocprofiler64.so.2"}, "1"), ({"COEUS_NO_GRAPH": "1"}, "0")]:
        env = {k: v for k, v in os.environ.items() if k not in ("HSA_TOOLS_LIB", "ROCP_TOOL_LIBRARIES")}
        env.update(extra)
        out = subprocess.run([sys.executable, "-c", code], env=env, cwd=root, capture_output=True, text=True)
        assert out.returncode == 0 and out.stdout.strip() == want, (extra, out.stdout, out.stderr[-400:])
