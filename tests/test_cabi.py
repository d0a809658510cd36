"""The C ABI without a device: the library loads, exports every symbol that
include/roller_hip.h declares, validates its arguments, JIT-compiles for gfx950 (hiprtc needs no
GPU) and maintains its on-disk code-object cache.  No compute call is made here."""

import ctypes as C
import re
from pathlib import Path

import pytest

from mlir_roller_amd import hip
from mlir_roller_amd.hip import GemmConfig, HipError

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "roller_hip.h").read_text()


def declared_functions():
    body = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    return sorted(set(re.findall(r"\b(rl_[a-z0-9_]+)\s*\(", body)))


def test_every_declared_symbol_is_exported(hip_lib):
    names = declared_functions()
    assert len(names) >= 35 and "rl_gemm_f32" in names and "rl_launch" in names
    for name in names:
        assert hasattr(hip_lib, name), f"{name} declared in roller_hip.h but not exported"
    # and the binding knows every one of them (argument types set, nothing bound by accident)
    assert sorted(hip.EXPORTS) == names


def test_every_declaration_cites_the_reference_or_says_why_not():
    # each block comment in the ABI section names a reference file:line
    assert HEADER.count("src/roller.py:") >= 10 and "src/arch.py:" in HEADER and "benchmark.py:" in HEADER


def test_config_struct_agrees_in_header_binding_and_documented_stub():
    # rl_gemm_config is passed by pointer: a binding with fewer fields makes the library read past it
    struct = re.search(r"typedef struct rl_gemm_config\s*\{(.*?)\}\s*rl_gemm_config;", HEADER, flags=re.S).group(1)
    struct = re.sub(r"/\*.*?\*/", "", struct, flags=re.S)
    in_header = [name for decl in re.findall(r"\bint\s+([a-z_,\s]+);", struct) for name in re.findall(r"[a-z_]+", decl)]
    in_binding = [name for name, _ in hip._GemmConfigC._fields_]
    in_dataclass = [f.name for f in __import__("dataclasses").fields(GemmConfig)]
    assert in_header == in_binding == in_dataclass and in_header[-3:] == ["direct", "trans_b", "streamk"]
    # the binding stubs that the repository's documents show to maintainers of the reference
    docs = [p.read_text() for p in sorted(ROOT.glob("*.md"))]
    doc = next(d for d in docs if "class GemmConfig(C.Structure)" in d)
    stub = re.search(r"for n in \((.*?)\)\]", doc, flags=re.S).group(1)
    assert re.findall(r'"([a-z_]+)"', stub) == in_header
    # the literal configs of the document are accepted by the library's own validation
    py_literal = re.search(r"cfg\s*=\s*GemmConfig\(([^)]*)\)", doc).group(1)
    hip.config_check(GemmConfig(*[int(v) for v in py_literal.split(",")]))
    c_literal = re.search(r"rl_gemm_config cfg = \{(.*?)\};", doc, flags=re.S).group(1)
    hip.config_check(GemmConfig(**{k: int(v) for k, v in re.findall(r"\.([a-z_]+)=(\d+)", c_literal)}))


def test_template_source_is_embedded_verbatim(hip_lib):
    # what the JIT compiles: the work decomposition of the stream-K variant, then the template
    csrc = ROOT / "mlir-roller_amd" / "csrc"
    on_disk = (csrc / "gemm_f32_mfma.hip").read_text()
    assert hip.template_source() == (csrc / "gemm_sk_decode.inc").read_text() + "\n" + on_disk
    assert 'extern "C" __global__' in on_disk and "gemm_kernel" in on_disk


def test_config_check_accepts_and_sizes(hip_lib):
    lds, threads = hip.config_check(GemmConfig(256, 256, 32, 128, 128, 32, 2, 4, 0, 4, 0))
    assert threads == 256 and lds == 2 * (256 * 36 + 32 * 256) * 4
    cfg = GemmConfig(128, 128, 16, 64, 64)
    assert hip.config_check(cfg) == (cfg.lds_bytes, cfg.threads)


@pytest.mark.parametrize("bad,needle", [
    (dict(mi=8), "mi must be"),
    (dict(wm=48), "does not divide block tile"),
    (dict(wm=64, wn=64, bm=64, bn=64, mi=32, bk=12), "bk must be a multiple"),
    (dict(stages=6), "stages must be"),
    (dict(stages=4), "needs direct=1"),
    (dict(stages=4, direct=1, pad_a=0, bm=32, bn=64, wm=32, wn=32, bk=8), "multiples of the 128 threads"),
    (dict(stages=5, direct=1, pad_a=0, bm=256, bn=256, wm=128, wn=128, bk=32), "exceed the 160 KB"),
    (dict(vec=2), "vec must be"),
    (dict(pad_a=2), "pad_a/pad_b"),
    (dict(bm=512, bn=512, wm=128, wn=128, bk=64), "exceed"),
    (dict(bm=1024, bn=1024, wm=32, wn=32, bk=8), "threads per workgroup"),
    (dict(edge=3), "edge is 0, 1 or 2"),
    (dict(accum=2), "accum is 0 or 1"),
    (dict(mi=16, bk=8), "bk must be a multiple of 16"),
    (dict(direct=1), "direct=1 needs stages>=3"),
    (dict(direct=1, stages=3, pad_a=0, vec=1, edge=2), "direct=1 with vec=1 (dword-aligned rows) needs stages=3 and edge=1"),
    (dict(direct=1, stages=4, pad_a=0, vec=1, edge=1, bk=32), "direct=1 with vec=1 (dword-aligned rows) needs stages=3 and edge=1"),
    (dict(direct=2), "direct is 0 or 1"),
    (dict(direct=1, stages=3, pad_a=0, bk=24), "power of two"),
])
def test_config_check_rejects(hip_lib, bad, needle):
    with pytest.raises(HipError) as err:
        hip.config_check(GemmConfig(**bad))
    assert err.value.status == hip.RL_ERR_INVALID_ARG and needle in str(err.value)


def test_config_check_accepts_any_column_block_count(hip_lib):
    # 3, 5, 6, 10 column blocks per wave: read with dword / 64-bit loads instead of 128-bit ones
    for cfg in (GemmConfig(96, 96, 16, 96, 96), GemmConfig(192, 320, 32, 96, 160, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1),
                GemmConfig(192, 320, 32, 48, 160, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1), GemmConfig(96, 96, 16, 48, 48, 16)):
        assert hip.config_check(cfg) == (cfg.lds_bytes, cfg.threads)


def test_config_check_limits_mfma_blocks_per_wave(hip_lib):
    hip.config_check(GemmConfig(256, 128, 32, 128, 64, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1))        # 8 x 4 blocks
    with pytest.raises(HipError, match="at most 32"):
        hip.config_check(GemmConfig(256, 256, 32, 128, 128, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1))   # 8 x 8 blocks
    with pytest.raises(HipError, match="32 MFMA blocks"):
        hip.compile_source(hip.template_source(), "gemm.hip", ["-DBM=256", "-DBN=256", "-DWM=128", "-DWN=128", "-DMI=16", "-DBK=32"])


def test_compile_plain_source_without_gpu(hip_lib):
    code, log = hip.compile_source('extern "C" __global__ void k(float* p) { p[threadIdx.x] = 1.0f; }', "k.hip")
    assert code[:4] == b"\x7fELF" and len(code) > 1000
    with pytest.raises(HipError) as err:
        hip.compile_source('extern "C" __global__ void k(float* p) { p[0] = undefined_symbol; }', "bad.hip")
    assert err.value.status == hip.RL_ERR_COMPILE and "undefined_symbol" in str(err.value)


def test_template_compiles_for_both_mfma_shapes(hip_lib):
    src = hip.template_source()
    for mi, bk in ((32, 16), (16, 16)):
        code, _ = hip.compile_source(src, "gemm.hip", [f"-DMI={mi}", f"-DBK={bk}", "-DEDGE=1"])
        assert b"gemm_kernel" in code
    # a configuration the template must refuse at compile time
    with pytest.raises(HipError) as err:
        hip.compile_source(src, "gemm.hip", ["-DBM=128", "-DWM=48"])
    assert "wave tile must divide block tile" in str(err.value)


def test_precompile_fills_the_disk_cache(hip_lib, tmp_path):
    try:
        hip.set_cache_dir(tmp_path)
        cfg = GemmConfig(64, 64, 16, 32, 32, 32, 2, 4, 0, 4, 1)
        size = hip.precompile(cfg)
        files = list(tmp_path.glob("gemm_*.hsaco"))
        assert len(files) == 1 and files[0].stat().st_size == size + 16               # code object + checksum trailer
        stamp = files[0].stat().st_mtime_ns
        assert hip.precompile(cfg) == size and files[0].stat().st_mtime_ns == stamp   # cache hit: not rewritten
        good = files[0].read_bytes()
        for damaged in (b"not a code object", good[:-1], good[:100] + bytes([good[100] ^ 1]) + good[101:]):
            files[0].write_bytes(damaged)                                                # fails the checksum: replaced
            assert hip.precompile(cfg) == size and files[0].read_bytes() == good
        hip.precompile(GemmConfig(64, 64, 16, 32, 32, 32, 2, 4, 0, 4, 0))
        assert len(list(tmp_path.glob("gemm_*.hsaco"))) == 2                             # key covers every field
        hip.set_cache_dir(None)
        with pytest.raises(HipError) as err:
            hip.precompile(cfg)
        assert err.value.status == hip.RL_ERR_IO
    finally:
        hip.set_cache_dir(hip.DEFAULT_CACHE_DIR)


def test_null_arguments_are_errors_not_crashes(hip_lib):
    assert hip_lib.rl_gemm_config_check(None, None, None) == hip.RL_ERR_INVALID_ARG
    assert hip_lib.rl_device_info(None) == hip.RL_ERR_INVALID_ARG
    assert hip_lib.rl_gemm_plan_launch(None, None, None, None, 1, 1, 1, 1, 1, 1, None) == hip.RL_ERR_INVALID_ARG
    assert hip_lib.rl_launch(None, 1, 1, 1, 1, 1, 1, 0, None, None, 0) == hip.RL_ERR_INVALID_ARG
    assert hip_lib.rl_event_record(None, None) == hip.RL_ERR_INVALID_ARG
    assert b"NULL" in hip_lib.rl_last_error()
    assert hip_lib.rl_free(None) == 0 and hip_lib.rl_module_unload(None) == 0   # freeing nothing is fine
    assert hip_lib.rl_gemm_plan_lds_bytes(None) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(hip, "_lib", None)
    monkeypatch.setattr(hip, "LIB_PATH", tmp_path / "libroller_hip.so")
    with pytest.raises(HipError) as err:
        hip.lib()
    assert "missing" in str(err.value)


def test_concurrent_precompiles_and_thread_local_errors(hip_lib, tmp_path):
    """ctypes releases the GIL inside the library: eight threads compile into one cache directory and
    provoke errors at the same time; every thread sees its own error text and every entry is intact."""
    import threading
    results, errors = {}, {}

    def work(i):
        try:
            cfg = GemmConfig(64, 64, 16, 32, 32, 32, 1 + i % 3, 4, 0, 4, i % 2)
            results[i] = hip.precompile(cfg)
            try:
                hip.config_check(GemmConfig(64, 64, 16, 32, 32, 32, 2, 4, 0, 4 + i, 0))     # vec = 4 + i is invalid
            except HipError as e:
                errors[i] = str(e)
        except Exception as e:                                                              # pragma: no cover
            errors[i] = f"unexpected: {e!r}"

    try:
        hip.set_cache_dir(tmp_path)
        threads = [threading.Thread(target=work, args=(i,)) for i in range(1, 9)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=120)
        assert sorted(results) == list(range(1, 9)) and all(v > 1000 for v in results.values())
        for i in range(1, 9):
            assert f"got {4 + i}" in errors[i], errors[i]                                   # its own message, not a neighbour's
        files = list(tmp_path.glob("gemm_*.hsaco"))
        assert len(files) == 6 and not list(tmp_path.glob("*.tmp*"))                          # 3 depths x 2 edge modes
        for f in files:
            assert f.read_bytes()[:4] == b"\x7fELF" and f.read_bytes()[-16:-12] == b"RLHC"
    finally:
        hip.set_cache_dir(hip.DEFAULT_CACHE_DIR)


def test_lds_requests_beyond_a_cu_are_refused_without_a_device(hip_lib):
    # more dynamic LDS than a CU has: refused with text before anything reaches the runtime
    assert hip_lib.rl_func_set_max_dynamic_lds(C.c_void_p(1), 160 * 1024 + 4) == hip.RL_ERR_INVALID_ARG
    assert b"exceed the 160 KB" in hip_lib.rl_last_error()
    assert hip_lib.rl_func_set_max_dynamic_lds(None, 1024) == hip.RL_ERR_INVALID_ARG
    with pytest.raises(HipError, match="exceed the 160 KB"):
        hip.config_check(GemmConfig(256, 256, 48, 128, 128, 32, 2, 0, 0, 4, 1))       # 2 x 96 KB
    assert hip_lib.rl_gemm_plan_lds_limit(None) == 0 and hip_lib.rl_gemm_plan_lds_bytes(None) == 0
