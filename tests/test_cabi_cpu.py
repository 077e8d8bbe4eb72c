"""Host-side checks that need no GPU: the C ABI library loads, exports every
symbol the headers declare, and validates layer descriptions the way the
boundary documents (capacity -> hipErrorUnknown before any pointer is looked
at, as the reference's API test expects of CreateLauncher)."""
import ctypes
import os
import re

import pytest

from flash_distributed_moe_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    names = set()
    for fn in ("flash_moe.h", "iMoeKernelLauncher.h"):
        text = open(os.path.join(ROOT, "include", fn)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        names |= set(re.findall(r"\b(flashMoe\w+)\s*\(", text))
        names |= set(re.findall(r'extern "C"[^;]*?\b(\w+)\s*\(', text))
    return names


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = header_symbols()
    assert {"flashMoeCreate", "flashMoeLaunch", "flashMoeDestroy", "CreateLauncher",
            "DestroyLauncher", "GetDistributedUniqueId", "CreateLauncherEx"} <= declared
    for name in sorted(declared):
        assert hasattr(lib, name), "libflashMoe.so does not export " + name
    assert set(_lib.C_ABI) | set(_lib.CXX_ABI) == declared
    assert b"gfx950" in lib.flashMoeVersion()


def desc(**kw):
    d = _lib.LayerDesc()
    d.experts, d.hidden, d.intermediate, d.top_k = 128, 2048, 768, 8
    d.dtype, d.max_tokens, d.sched = _lib.BF16, 64, 0
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def workspace(d):
    n = ctypes.c_size_t(0)
    rc = _lib.load().flashMoeWorkspaceBytes(ctypes.byref(d), ctypes.byref(n))
    return rc, n.value


def test_workspace_size_grows_with_tokens():
    rc1, n1 = workspace(desc(max_tokens=64))
    rc2, n2 = workspace(desc(max_tokens=8192))
    assert rc1 == 0 and rc2 == 0 and n2 > n1 > 0
    rows = 8192 * 8
    # at prefill sizes h [T*k, I] and y [T*k, H], both bf16, dominate (the tiled variant's)
    assert rows * (768 + 2048) * 2 <= n2 < rows * (768 + 2048) * 2 + (32 << 20)
    # the streaming variant alone keeps float rows of y for every (token, slot)
    rc3, n3 = workspace(desc(max_tokens=8192, sched=_lib.SCHED_STREAM))
    assert rc3 == 0 and n3 >= rows * 2048 * 4


def test_workspace_of_the_optional_steps_and_weight_modes():
    base = workspace(desc(max_tokens=4096))[1]
    # the normalised rows live in the workspace: max_tokens x H elements, no more
    with_norm = workspace(desc(max_tokens=4096, flags=_lib.FLAG_RMSNORM))[1]
    assert 4096 * 2048 * 2 <= with_norm - base < 4096 * 2048 * 2 + 4096
    # the residual needs nothing; weights the caller packed in place need nothing either
    assert workspace(desc(max_tokens=4096, flags=_lib.FLAG_RESIDUAL))[1] == base
    assert workspace(desc(max_tokens=64, flags=_lib.FLAG_WEIGHTS_PREPACKED))[1] == workspace(desc())[1]
    # the launcher's own packed copy is the size of the expert weights
    copy = workspace(desc(flags=_lib.FLAG_PACK_WEIGHTS))[1] - workspace(desc())[1]
    assert 3 * 128 * 2048 * 768 * 2 <= copy < 3 * 128 * 2048 * 768 * 2 + 4096
    # unknown flag bits, and the two weight modes together, are refused
    assert workspace(desc(flags=16))[0] == _lib.HIP_ERROR_INVALID_VALUE
    assert workspace(desc(flags=_lib.FLAG_PACK_WEIGHTS | _lib.FLAG_WEIGHTS_PREPACKED))[0] == \
        _lib.HIP_ERROR_INVALID_VALUE


@pytest.mark.parametrize("kw", [
    dict(experts=0), dict(experts=257), dict(top_k=0), dict(top_k=129), dict(top_k=33),
    dict(hidden=2000), dict(hidden=0), dict(intermediate=100), dict(dtype=7),
    dict(max_tokens=0), dict(sched=9),
])
def test_bad_descriptions_are_invalid_value(kw, capfd):
    rc, _ = workspace(desc(**kw))
    assert rc == _lib.HIP_ERROR_INVALID_VALUE
    assert "[MOE ERROR:" in capfd.readouterr().out    # printed to stdout, reference convention


def test_capacity_is_hip_error_unknown_before_pointers(capfd):
    # null weights everywhere: capacity is still what is reported
    d = desc(max_tokens=(1 << 21) // 8 + 1)
    rc, _ = workspace(d)
    assert rc == _lib.HIP_ERROR_UNKNOWN
    h = ctypes.c_void_p()
    rc = _lib.load().flashMoeCreate(ctypes.byref(h), ctypes.byref(d), None)
    assert rc == _lib.HIP_ERROR_UNKNOWN and not h.value
    assert "beyond capacity" in capfd.readouterr().out


def test_null_weights_are_invalid_value_and_result_untouched():
    d = desc()
    h = ctypes.c_void_p(0x1234)
    rc = _lib.load().flashMoeCreate(ctypes.byref(h), ctypes.byref(d), None)
    assert rc == _lib.HIP_ERROR_INVALID_VALUE and h.value == 0x1234


def test_python_launcher_surface():
    from flash_distributed_moe_amd.flashMoeLauncher import MoeKernelLauncher

    l = MoeKernelLauncher()
    assert l.valid is False
    uid = l.getDistributedUniqueId(empty=True)
    assert isinstance(uid, bytes) and len(uid) == 128 and uid == bytes(128)
    with pytest.raises(RuntimeError, match="Launcher was destroyed"):
        l.launch(None, None)
    l.destroy()                       # destroying an empty launcher is a no-op
    assert l.valid is False


def test_drop_in_python_module_imports_by_the_reference_name():
    """`import flashMoeLauncher` (test/singleGPU/python/flashMoeOp.py:1,
    test_pythonBinding.py:2 of the reference) resolves to the compiled extension."""
    import flashMoeLauncher

    assert flashMoeLauncher.__file__.endswith(".so")
    l = flashMoeLauncher.MoeKernelLauncher()
    assert l.valid is False
    uid = l.getDistributedUniqueId(empty=True)
    assert isinstance(uid, bytes) and uid == bytes(128)
    l.destroy()                       # a no-op on an empty launcher
    assert l.valid is False
