"""The structs that cross the C ABI have one layout: what the C compiler gives
include/coeus.h's declarations (sizeof / offsetof printed by a small C program compiled here) is
what ctypes computes for coeus_amd/_lib.py's mirrors, and what #[repr(C)] gives the Rust shim's
mirror (bindings/rust/.../src/lib.rs cannot be compiled in this image, so its field list is parsed
and laid out by the repr(C) rule: every field at the next multiple of its alignment, the size a
multiple of the largest alignment).  Also here: coeus_last_error is per thread."""
import ctypes as C
import os
import re
import subprocess
import threading

from coeus_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RUST = os.path.join(ROOT, "bindings", "rust", "model-transformer-mi355x", "src", "lib.rs")

CONFIG_FIELDS = ["hidden_dim", "num_layers", "num_heads", "intermediate_dim", "vocab_size", "max_seq_len",
                 "dropout", "attention_dropout", "layer_norm_eps", "use_bias", "activation", "norm",
                 "norm_scope", "weight_dtype", "kv_dtype", "head_dim", "max_batch"]
SAMPLING_FIELDS = ["temperature", "top_k", "top_p", "seed"]


def c_layout(tmp_path):
    lines = ['#include <stddef.h>', '#include <stdio.h>', '#include "coeus.h"', 'int main(void) {',
             '  printf("coeus_config %zu %zu\\n", sizeof(coeus_config), _Alignof(coeus_config));',
             '  printf("coeus_sampling %zu %zu\\n", sizeof(coeus_sampling), _Alignof(coeus_sampling));']
    for f in CONFIG_FIELDS:
        lines.append(f'  printf("coeus_config.{f} %zu %zu\\n", offsetof(coeus_config, {f}), sizeof(((coeus_config *)0)->{f}));')
    for f in SAMPLING_FIELDS:
        lines.append(f'  printf("coeus_sampling.{f} %zu %zu\\n", offsetof(coeus_sampling, {f}), sizeof(((coeus_sampling *)0)->{f}));')
    lines += ['  return 0;', '}']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    out = {}
    for line in subprocess.check_output([str(exe)], text=True).splitlines():
        name, a, b = line.split()
        out[name] = (int(a), int(b))
    return out


def test_ctypes_mirrors_match_the_header(tmp_path):
    lay = c_layout(tmp_path)
    for cls, cname, fields in [(_lib.CConfig, "coeus_config", CONFIG_FIELDS), (_lib.CSampling, "coeus_sampling", SAMPLING_FIELDS)]:
        assert [f for f, _ in cls._fields_] == fields
        assert (C.sizeof(cls), C.alignment(cls)) == lay[cname]
        for f in fields:
            d = getattr(cls, f)
            assert (d.offset, d.size) == lay[f"{cname}.{f}"], (cname, f)
    # the figures the Rust file states next to its struct
    assert lay["coeus_config"] == (104, 8) and lay["coeus_config.use_bias"] == (60, 1)
    assert lay["coeus_config.activation"] == (64, 4) and lay["coeus_config.head_dim"] == (88, 8)


RUST_TYPES = {"u64": 8, "u32": 4, "u16": 2, "u8": 1, "f32": 4, "f64": 8, "i32": 4, "i64": 8}


def rust_repr_c_layout(struct_name):
    text = open(RUST).read()
    m = re.search(r"#\[repr\(C\)\][^{]*?pub struct " + struct_name + r"\s*\{(.*?)\n\}", text, flags=re.S)
    assert m, f"{struct_name} not found in the Rust shim"
    body = re.sub(r"//[^\n]*", "", m.group(1))
    off, align, out = 0, 1, {}
    for name, ty in re.findall(r"(\w+)\s*:\s*(\w+)\s*,", body):
        size = RUST_TYPES[ty]
        off = (off + size - 1) // size * size
        out[name] = (off, size)
        off += size
        align = max(align, size)
    return out, ((off + align - 1) // align * align, align)


def test_rust_mirror_matches_the_header(tmp_path):
    lay = c_layout(tmp_path)
    fields, total = rust_repr_c_layout("CoeusConfig")
    assert list(fields) == CONFIG_FIELDS  # same fields, same order
    assert total == lay["coeus_config"]
    for f in CONFIG_FIELDS:
        assert fields[f] == lay[f"coeus_config.{f}"], f
    # the constants written next to the struct (compile-time assertions in the Rust source)
    text = open(RUST).read()
    stated = dict(re.findall(r"const COEUS_CONFIG_(\w+): usize = (\d+);", text))
    assert int(stated["SIZE"]) == lay["coeus_config"][0]
    assert int(stated["OFFSET_USE_BIAS"]) == lay["coeus_config.use_bias"][0]
    assert int(stated["OFFSET_ACTIVATION"]) == lay["coeus_config.activation"][0]
    assert int(stated["OFFSET_HEAD_DIM"]) == lay["coeus_config.head_dim"][0]


def test_last_error_is_thread_local():
    """A failing call leaves its message for the calling thread only (coeus.h: thread-local, valid
    until the next failing call on that thread)."""
    lib = _lib.load()
    bad_layers, bad_vocab = _lib.CConfig(), _lib.CConfig()
    lib.coeus_config_default(C.byref(bad_layers))
    lib.coeus_config_default(C.byref(bad_vocab))
    bad_layers.num_layers = 0
    bad_vocab.vocab_size = 0
    seen, barrier = {}, threading.Barrier(3)

    def worker(name, cfg, want):
        ok = True
        for _ in range(200):
            assert lib.coeus_config_validate(C.byref(cfg)) == _lib.INVALID_CONFIG
            ok &= want in _lib.last_error()
        seen[name] = ok
        barrier.wait()

    def quiet():
        seen["quiet"] = _lib.last_error()  # a thread that never failed sees no message
        barrier.wait()

    ts = [threading.Thread(target=worker, args=("layers", bad_layers, "Number of layers")),
          threading.Thread(target=worker, args=("vocab", bad_vocab, "Vocabulary size")),
          threading.Thread(target=quiet)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert seen == {"layers": True, "vocab": True, "quiet": ""}


# ------------------------------------------------------------------ the Rust shim's extern declarations
# The shim cannot be compiled in this image, so every `fn coeus_*` it declares in an extern "C"
# block is parsed and compared with the declaration of the same name in include/coeus.h: same
# number of parameters, each Rust type the FFI equivalent of the C type, same return type.

RUST_TO_C = {
    "u64": "uint64_t", "u32": "uint32_t", "u8": "uint8_t", "f32": "float", "c_int": "int", "c_char": "char",
    "CoeusConfig": "coeus_config", "CoeusModel": "coeus_model", "CoeusBpe": "coeus_bpe",
    "CoeusSession": "coeus_session", "CoeusSampling": "coeus_sampling", "c_void": "void",
}


def rust_type_to_c(t):
    """Rust FFI type -> (C base type, pointer depth, innermost pointee is const)."""
    t = t.strip()
    depth, const = 0, False
    while True:
        m = re.fullmatch(r"\*(const|mut)\s+(.*)", t)
        if not m:
            break
        depth += 1
        const = m.group(1) == "const"  # the innermost qualifier is the last one seen
        t = m.group(2).strip()
    return (RUST_TO_C[t], depth, const if depth else False)


def normalise_c(t):
    """C type -> the same triple (`const char *const *` = char, 2, const)."""
    t = re.sub(r"\s+", " ", t.strip())
    depth = t.count("*")
    head = t.split("*", 1)[0].strip()
    const = bool(re.search(r"\bconst\b", head)) and depth > 0
    base = re.sub(r"\bconst\b", "", head).strip()
    return (base, depth, const)


def c_declarations():
    text = open(os.path.join(ROOT, "include", "coeus.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for ret, name, args in re.findall(r"([A-Za-z_][\w\s\*]*?)\b(coeus_\w+)\s*\(([^)]*)\)\s*;", text):
        params = []
        for a in [x for x in args.split(",") if x.strip() and x.strip() != "void"]:
            a = a.strip()
            a = re.sub(r"\b\w+$", "", a).strip() if not a.endswith("*") else a  # drop the parameter name
            params.append(normalise_c(a))
        out[name] = (normalise_c(ret), params)
    return out


def rust_declarations():
    decls = {}
    src = os.path.dirname(RUST)
    for f in sorted(os.listdir(src)):
        text = re.sub(r"//[^\n]*", "", open(os.path.join(src, f)).read())
        for block in re.findall(r'extern\s+"C"\s*\{(.*?)\n\}', text, flags=re.S):
            for name, args, ret in re.findall(r"fn\s+(coeus_\w+)\s*\(([^)]*)\)\s*(?:->\s*([^;]+))?;", block, flags=re.S):
                params = [rust_type_to_c(a.split(":", 1)[1]) for a in args.split(",") if a.strip()]
                decls.setdefault(name, []).append((rust_type_to_c(ret) if ret else ("void", 0, False), params, f))
    return decls


def test_rust_extern_declarations_match_the_header():
    c, r = c_declarations(), rust_declarations()
    assert len(r) >= 18
    for name, variants in r.items():
        assert name in c, f"the Rust shim binds {name}, which include/coeus.h does not declare"
        c_ret, c_params = c[name]
        for ret, params, f in variants:
            assert ret == c_ret, (f, name, ret, c_ret)
            assert params == c_params, (f, name, params, c_params)
