"""CPU-side checks of the C-ABI library and the host mirror: the shared object loads,
exports every symbol include/nabla_optim.h declares, and fails loudly (never
computes) without a gfx950 device.  No kernel is launched here."""
import ctypes as C
import os
import re

import pytest

from nabla_amd import _lib
from nabla_amd import optim as nb

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "nabla_optim.h")
BENCH_HEADER = os.path.join(ROOT, "include", "nabla_optim_bench.h")


def _declared_symbols(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nbo_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 30
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in nabla_optim.h but not exported"
    assert sorted(_lib.SYMBOLS) == declared, "ctypes table and header disagree"


def test_measurement_symbols_live_in_a_header_of_their_own():
    """The drop-in header declares only what replaces a reference interface (plus the
    allocation-free step); timing and memory-system probes are in nabla_optim_bench.h."""
    lib = _lib.load()
    bench = _declared_symbols(BENCH_HEADER)
    assert sorted(_lib.BENCH_SYMBOLS) == bench, "ctypes table and bench header disagree"
    for name in bench:
        assert hasattr(lib, name), f"{name} is declared in nabla_optim_bench.h but not exported"
    assert not set(bench) & set(_declared_symbols()), "a measurement symbol is declared in the drop-in header"
    for word in ("probe", "profile", "ceiling", "copy_bytes"):
        assert word not in re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)


def test_struct_layouts_match_the_header():
    assert C.sizeof(_lib.Meta) == 8 + 6 * 8 + 8
    assert C.sizeof(_lib.ScalerState) == 5 * 8
    assert C.sizeof(_lib.StepInfo) == 3 * 8 + 2 * 4


def test_version_and_status_strings():
    lib = _lib.load()
    assert lib.nbo_version().decode() == "0.1.0"
    assert lib.nbo_status_string(0) == b"ok"
    assert b"length mismatch" in lib.nbo_status_string(_lib.ERR_LEN_MISMATCH)
    assert b"kind mismatch" in lib.nbo_status_string(_lib.ERR_KIND)
    assert b"HIP" in lib.nbo_status_string(_lib.ERR_HIP + 2)


def _no_gpu():
    try:
        import torch

        return not torch.cuda.is_available()
    except Exception:
        return True


@pytest.mark.skipif(not _no_gpu(), reason="checks the behaviour without a GPU")
def test_no_device_is_an_error_not_a_fallback():
    lib = _lib.load()
    assert lib.nbo_init() == _lib.ERR_NO_DEVICE
    assert b"gfx950" in lib.nbo_last_error()
    with pytest.raises(_lib.NablaOptimError):
        _lib.init()
    # every object constructor needs the runtime and therefore fails the same way
    h = C.c_void_p()
    rows = (C.c_uint64 * 1)(1)
    meta = _lib.Meta(_lib.KIND_SGD, 0, 0.1, 0, 0, 0, 0, 0, 0)
    assert lib.nbo_optim_create(C.byref(meta), 1, rows, rows, _lib.DT_F32, 0, C.byref(h)) == \
        _lib.ERR_NO_DEVICE
    assert not h.value
    assert lib.nbo_scaler_create(None, C.byref(h)) == _lib.ERR_NO_DEVICE


def test_argument_errors_are_reported_before_any_device_work():
    lib = _lib.load()
    assert lib.nbo_optim_create(None, 0, None, None, _lib.DT_F32, 0, None) == _lib.ERR_ARG
    assert lib.nbo_optim_step(None, None, None) == _lib.ERR_ARG
    assert lib.nbo_zero_grad(None) == _lib.ERR_ARG
    out = C.c_double()
    assert lib.nbo_clip_grad_norm(None, 1.0, C.byref(out)) == _lib.ERR_ARG
    assert lib.nbo_list_destroy(None) in (_lib.OK, _lib.ERR_NO_DEVICE)


# ---- host mirror: the parts of OptimState that are plain string / key logic -----------------

def test_rust_f64_display():
    """Rust's Display for f64 (used by optim_meta_pairs, core.rs:263-277): shortest
    round-trip digits, no exponent, integers without a fraction."""
    f = nb.rust_f64_str
    assert f(1e-8) == "0.00000001"
    assert f(0.1) == "0.1" and f(0.9) == "0.9" and f(0.999) == "0.999"
    assert f(65536.0) == "65536" and f(0.0) == "0" and f(2.0) == "2"
    assert f(3e-4) == "0.0003" and f(2e-4) == "0.0002"
    assert f(1e21) == "1000000000000000000000"
    assert f(-1.5e-7) == "-0.00000015"
    assert f(float("inf")) == "inf" and f(float("nan")) == "NaN"
    for x in (1e-8, 3e-4, 0.95, 123456.789, 1e-300, 1.7976931348623157e308):
        assert float(f(x)) == x


def test_meta_pairs_round_trip_and_errors():
    meta = nb.OptimMeta("adamw", 2e-4, 0.9, 0.95, 1e-8, 0.1, 0.0, 48)
    pairs = nb.optim_meta_pairs(meta)
    assert pairs[0] == ("optim.kind", "adamw") and pairs[4] == ("optim.eps", "0.00000001")
    assert pairs[-1] == ("optim.step_count", "48")
    assert nb.parse_optim_meta(dict(pairs)) == meta
    m = dict(pairs)
    del m["optim.beta2"]
    with pytest.raises(nb.OptimStateError, match="missing optim.beta2"):
        nb.parse_optim_meta(m)
    m = dict(pairs, **{"optim.kind": "lion"})
    with pytest.raises(nb.OptimStateError, match="bad optim.kind: lion"):
        nb.parse_optim_meta(m)
    m = dict(pairs, **{"optim.step_count": "-3"})
    with pytest.raises(nb.OptimStateError, match="bad optim.step_count: -3"):
        nb.parse_optim_meta(m)
    m = dict(pairs, **{"optim.lr": "fast"})
    with pytest.raises(nb.OptimStateError, match="bad optim.lr: fast"):
        nb.parse_optim_meta(m)


def test_load_state_tensors_key_errors_follow_the_reference():
    """alg.rs:487-516: checks run before anything is written, so no device is needed."""
    opt = nb.AdamW.new(1e-3, [(1, 1), (2, 2)])
    with pytest.raises(nb.OptimStateError, match="bad tensor key: mx"):
        opt.load_state_tensors([("mx", None)])
    with pytest.raises(nb.OptimStateError, match="m index out of range: 2"):
        opt.load_state_tensors([("m2", None)])
    with pytest.raises(nb.OptimStateError, match="missing m0"):
        opt.load_state_tensors([("m1", None), ("v0", None), ("v1", None), ("other", None)])
    with pytest.raises(nb.OptimStateError, match="missing v1"):
        opt.load_state_tensors([("m0", None), ("m1", None), ("v0", None)])
    sgd = nb.Sgd.new(0.1, [(1, 1)])
    with pytest.raises(nb.OptimStateError, match="missing v0"):
        sgd.load_state_tensors([("m0", None)])  # Sgd ignores every prefix but 'v'
    with pytest.raises(nb.OptimStateError, match="optim kind mismatch"):
        sgd.load_meta(nb.OptimMeta("adam", 0.1, 0.9, 0.999, 1e-8, 0.0, 0.0, 0))


def test_meta_before_first_use_reports_constructor_defaults():
    """alg.rs:29-38, 190-198, 324-329 and the zeros each kind's meta() reports."""
    a = nb.AdamW.new(2e-4, [(1, 1)]).beta2(0.95).weight_decay(0.1).meta()
    assert (a.kind, a.lr, a.beta1, a.beta2, a.eps, a.weight_decay, a.momentum, a.step_count) == \
        ("adamw", 2e-4, 0.9, 0.95, 1e-8, 0.1, 0.0, 0)
    d = nb.Adam.new(3e-4, [(1, 1)]).meta()
    assert (d.kind, d.beta2, d.weight_decay) == ("adam", 0.999, 0.0)
    s = nb.Sgd.new(0.01, [(1, 1)]).momentum(0.9).meta()
    assert (s.kind, s.beta1, s.eps, s.momentum, s.step_count) == ("sgd", 0.0, 0.0, 0.9, 0)
    g = nb.GradScaler.new().state()
    assert (g.scale, g.growth_factor, g.backoff_factor, g.growth_interval, g.consecutive_ok) == \
        (65536.0, 2.0, 0.5, 2000, 0)


class _Module:
    def __init__(self, params):
        self._p = params

    def parameters_mut(self):
        return self._p


class _Var:
    def __init__(self, grad):
        self._g = grad

    def grad(self):
        if self._g is None:
            raise RuntimeError("no grad")
        return self._g


def test_step_with_vars_panics_like_the_reference():
    """optim/core.rs:18-39: both asserts fire before anything reaches the device."""
    opt = nb.Sgd.new(0.1, [(1, 1), (1, 1)])
    with pytest.raises(nb.NablaPanic, match=r"param_vars length \(1\) doesn't match module parameters count \(2\)"):
        opt.step_with_vars(_Module([object(), object()]), [_Var(object())])
    with pytest.raises(nb.NablaPanic, match=r"param_vars\[1\] has no gradient \(call backward first\)"):
        opt.step_with_vars(_Module([object(), object()]), [_Var(object()), _Var(None)])


def test_header_is_plain_c99_and_links_from_c(tmp_path):
    """The boundary is a C ABI: a C99 translation unit that includes the header compiles
    with -pedantic -Werror, links against the library and calls it."""
    import subprocess

    src = tmp_path / "t.c"
    src.write_text('#include "nabla_optim.h"\n#include <stdio.h>\n#include <string.h>\n'
                   "int main(void) {\n"
                   "    nbo_meta m; nbo_scaler_state s; nbo_step_info i;\n"
                   "    memset(&m, 0, sizeof m); memset(&s, 0, sizeof s); memset(&i, 0, sizeof i);\n"
                   '    printf("%s|%s|%d\\n", nbo_version(), nbo_status_string(NBO_ERR_KIND), (int)NBO_BACKEND_AXPY);\n'
                   "    return nbo_optim_step(0, 0, 0) == NBO_ERR_ARG ? 0 : 1;\n"
                   "}\n")
    exe = tmp_path / "t"
    libdir = os.path.join(ROOT, "nabla_amd")
    r = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
                        "-o", str(exe), str(src), "-L", libdir, "-l:libnabla_optim.so",
                        f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.strip() == "0.1.0|optim kind mismatch|1", r.stdout + r.stderr


def test_null_arguments_are_errors_not_crashes():
    """Every entry point checks its pointers before it touches the device: with nulls
    they return NBO_ERR_ARG and leave a message, with or without a GPU."""
    lib = _lib.load()
    null = None
    calls = [
        lambda: lib.nbo_list_create(1, null, null, 0, null, null),
        lambda: lib.nbo_list_set_ptrs(null, null),
        lambda: lib.nbo_optim_create(null, 0, null, null, 0, 0, null),
        lambda: lib.nbo_optim_step(null, null, null),
        lambda: lib.nbo_optim_reset(null),
        lambda: lib.nbo_optim_set_lr(null, 0.1),
        lambda: lib.nbo_optim_get_meta(null, null),
        lambda: lib.nbo_optim_load_meta(null, null),
        lambda: lib.nbo_optim_state_read(null, b"m0", null, 0, 0),
        lambda: lib.nbo_optim_state_write(null, b"m0", null, 0, 0),
        lambda: lib.nbo_optim_master_from_params(null, null),
        lambda: lib.nbo_optim_state_regions(null, null),
        lambda: lib.nbo_scaler_create(null, null),
        lambda: lib.nbo_scaler_state_get(null, null),
        lambda: lib.nbo_scaler_load_state(null, null),
        lambda: lib.nbo_scaler_unscale_and_update(null, null, null),
        lambda: lib.nbo_clip_grad_norm(null, 1.0, null),
        lambda: lib.nbo_has_non_finite(null, null),
        lambda: lib.nbo_zero_grad(null),
        lambda: lib.nbo_scale_grad(null, 1.0),
        lambda: lib.nbo_fused_step(null, null, null, null, 1.0, 0),
        lambda: lib.nbo_fused_step_groups(1, null, null, null, null, null, 1.0, 0),
        lambda: lib.nbo_accumulate(null, null, 0),
        lambda: lib.nbo_backend_apply(0, null, null, null, 1.0),
        lambda: lib.nbo_backend_apply(99, null, null, null, 1.0),
        lambda: lib.nbo_backend_cast(null, null),
        lambda: lib.nbo_optim_last_step(null, null),
        lambda: lib.nbo_optim_trace_read(null, null, 0, null, null),
        lambda: lib.nbo_nbla_save_list(b"/nonexistent/x", null, null),
        lambda: lib.nbo_nbla_load_list(b"/nonexistent/x", null, null),
        lambda: lib.nbo_optim_save_state(null, b"/nonexistent/x"),
        lambda: lib.nbo_optim_load_state(null, b"/nonexistent/x"),
        lambda: lib.nbo_copy_bytes(null, null, 16),
        lambda: lib.nbo_profile_read(null, null, null),
        lambda: lib.nbo_selftest_half_arith(1, null, null, null, null),
        lambda: lib.nbo_fused_step_noalloc(null, null, null, null, 1.0, 0),
        lambda: lib.nbo_fused_step_norm(null, null, null, 1.0, 1.0, 0),
        lambda: lib.nbo_unscale_accumulate(null, null, null, 0, null, null),
        lambda: lib.nbo_optim_state_placement_note(null, null, 0),
        lambda: lib.nbo_optim_save_master(null, b"/nonexistent/x", null),
        lambda: lib.nbo_optim_load_master(null, b"/nonexistent/x", null),
        lambda: lib.nbo_optim_params_from_master(null, null),
        lambda: lib.nbo_hbm_ceiling(0, 0, 1 << 20, 2, 0, null, null, null),
        lambda: lib.nbo_hbm_ceiling(99, 0, 1 << 20, 2, 0, null, null, null),
    ]
    for k, call in enumerate(calls):
        assert call() == _lib.ERR_ARG, f"call {k}"
        assert lib.nbo_last_error(), f"call {k} left no message"
    # destroying nothing is fine, as free(NULL) is
    assert lib.nbo_list_destroy(null) in (0, _lib.ERR_NO_DEVICE)


def test_placement_decisions_on_made_up_measurements(tmp_path):
    """The region search and the chunk assignment of the state placement are GPU-free functions
    (nabla_amd/csrc/host/nbo_placement_plan.hpp); tests/cpp/test_placement_plan.cpp drives them
    with a mocked bandwidth probe: three, two and one region, a noisy fourth kind, a failed
    probe, regions that run dry, exhaustion, a slower and a faster GPU."""
    import subprocess

    src = os.path.join(ROOT, "tests", "cpp", "test_placement_plan.cpp")
    exe = str(tmp_path / "test_placement_plan")
    subprocess.run(["g++", "-O1", "-std=c++17", "-Wall", "-Wextra", "-o", exe, src], check=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout
