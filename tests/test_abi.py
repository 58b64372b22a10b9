"""The C-ABI library loads and exports every symbol include/mamba_hip.h declares (no compute)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    names = []
    for fn in sorted(os.listdir(os.path.join(ROOT, "include"))):
        if fn.endswith(".h"):
            text = open(os.path.join(ROOT, "include", fn)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            names += re.findall(r"\bMRS_API\b[^;(]*?\b(mrs_\w+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    from mamba_rs_amd import _lib
    lib = _lib.load()
    names = header_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/ but not exported"
    # and the Python binding table covers exactly the header
    from mamba_rs_amd.backbone import engine_exported_names
    from mamba_rs_amd.mamba3 import m3_engine_exported_names
    assert sorted(_lib.exported_names() + engine_exported_names() + m3_engine_exported_names()) == names


def test_version_and_error_string_and_dispatch_predicate():
    from mamba_rs_amd import ScanMode, _lib
    lib = _lib.load()
    assert lib.mrs_version() >= 100
    assert isinstance(lib.mrs_last_error(), bytes)
    # ScanMode::use_parallel, tests/scan_mode_boundary.rs:12-53
    THR = 256
    assert not ScanMode.AUTO.use_parallel(THR - 1, 16)
    assert not ScanMode.AUTO.use_parallel(THR, 16)
    assert ScanMode.AUTO.use_parallel(THR + 1, 16)
    for mode in ScanMode:
        assert mode.use_parallel(1, 65)
    assert not ScanMode.SEQUENTIAL.use_parallel(1 << 20, 16)
    assert ScanMode.PARALLEL.use_parallel(1, 16)
    for mode in ScanMode:
        for t in (1, THR - 1, THR, THR + 1, 4621):
            for ds in (8, 16, 64, 65, 256):
                assert (mode.resolve(t, ds) == ScanMode.PARALLEL) == mode.use_parallel(t, ds)


def test_argument_errors_need_no_gpu():
    from mamba_rs_amd import MambaHipError, _lib
    with pytest.raises(MambaHipError) as e:
        _lib.call("mrs_exp_negate", None, None, None, 4)
    assert e.value.code == -1 and "null" in e.value.message


def test_static_scratch_scan_refuses_oversized_shapes_before_touching_a_gpu():
    """mrs_ssm_scan_fwd_static: a shape whose chunk summaries exceed the built-in buffer is refused by size alone."""
    from mamba_rs_amd import MambaHipError, _lib, ops
    assert _lib.load().mrs_ssm_scan_workspace_bytes(8, 2048, 1536, 16) <= ops.SCAN_STATIC_SCRATCH_BYTES
    assert _lib.load().mrs_ssm_scan_workspace_bytes(4, 4096, 5120, 16) <= ops.SCAN_STATIC_SCRATCH_BYTES
    with pytest.raises(MambaHipError) as e:
        _lib.call("mrs_ssm_scan_fwd_static", None, 2, 1, 1, 1, 1, 1, 1, 16, 1, 1, None, 0, 0, 40, 512, 4096, 16)
    assert e.value.code == -4 and "built-in buffer" in e.value.message


def test_config_validate_bounds():
    # src/config.rs:108-170
    from mamba_rs_amd import MambaConfig
    MambaConfig().validate()
    for bad in (dict(d_model=0), dict(d_state=257), dict(d_conv=9), dict(d_model=40000, expand=2), dict(d_model=3, expand=1),
                dict(n_layers=5000)):
        with pytest.raises(ValueError):
            MambaConfig(**bad).validate()
    c = MambaConfig(d_model=768)
    assert (c.d_inner(), c.dt_rank(), c.xdbl_dim()) == (1536, 48, 80)
