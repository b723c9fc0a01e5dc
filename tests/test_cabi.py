"""The C-ABI shared library loads and exports every symbol include/thip.h declares (no compute here)."""
import ctypes
import os
import re

import pytest

from torq_compiler_amd import ThipError, runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "thip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(thip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(runtime.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 35
    for name in names:
        assert hasattr(lib, name), "libthip.so does not export %s" % name
    assert sorted(runtime.EXPORTED_SYMBOLS) == names, "runtime.EXPORTED_SYMBOLS is out of date with include/thip.h"


def test_version_and_status_message():
    lib = runtime.lib()
    assert lib.thip_descriptor_version() == 2
    assert lib.thip_version() >= 1
    p = ctypes.c_void_p()
    assert lib.thip_program_create(ctypes.byref(p)) == runtime.OK
    blob, size = ctypes.c_void_p(), ctypes.c_size_t()
    code = lib.thip_program_serialize(p, ctypes.byref(blob), ctypes.byref(size))
    assert code == runtime.INVALID_ARGUMENT
    assert b"no ops" in lib.thip_status_message()
    lib.thip_program_destroy(p)


def test_null_arguments_are_rejected_not_dereferenced():
    lib = runtime.lib()
    assert lib.thip_program_create(None) == runtime.INVALID_ARGUMENT
    assert lib.thip_executable_run(None, None) == runtime.INVALID_ARGUMENT
    assert lib.thip_executable_create(None, None, 0, None, 0, None) == runtime.INVALID_ARGUMENT
    out = ctypes.c_void_p()
    assert lib.thip_executable_create(None, None, 0, None, 0, ctypes.byref(out)) == runtime.INVALID_ARGUMENT
    assert lib.thip_device_synchronize(None) == runtime.INVALID_ARGUMENT


def test_device_create_without_gpu_is_unavailable_or_ok():
    """No GPU in the build container: UNAVAILABLE with a message; on a GPU box: a gfx950 device."""
    try:
        dev = runtime.Device(0)
    except ThipError as e:
        assert e.code == runtime.UNAVAILABLE
        return
    assert dev.name() == "gfx950"
    dev.close()


def test_iree_glue_covers_every_op_entry_point():
    """The plugin-side serialiser (iree_glue/, built only inside the reference's tree) forwards every TorqHL op the
    C-ABI declares, and the HAL-side files call the run-side entry points they stand in front of."""
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    header = open(os.path.join(root, "include", "thip.h")).read()
    glue = open(os.path.join(root, "iree_glue", "ThipSerialization.cpp")).read()
    ops = sorted(set(re.findall(r"thip_status_t (thip_hl_\w+)\(", header)))
    assert len(ops) >= 13
    for name in ops:
        assert name + "(program_" in glue, name + " is not forwarded by iree_glue/ThipSerialization.cpp"
        assert name + "_t s = {}" in glue
    for name in ("thip_program_create", "thip_program_set_name", "thip_program_binding", "thip_program_constant", "thip_program_tensor",
                 "thip_program_serialize", "thip_blob_free", "thip_descriptor_validate"):
        assert name + "(" in glue, name
    hal = open(os.path.join(root, "iree_glue", "thip_native_executable.cc")).read() + open(os.path.join(root, "iree_glue", "thip_driver_module.c")).read()
    for name in ("thip_executable_create", "thip_executable_run", "thip_executable_destroy", "thip_infer_format", "thip_device_create", "thip_device_destroy"):
        assert name + "(" in hal, name
    # every iree_hal_thip_* symbol the glue calls is defined in the glue; every symbol of the reference's driver it
    # calls is named, with where it is declared, in the glue's README; every thip_* call is a symbol of the C-ABI
    gdir = os.path.join(root, "iree_glue")
    sources = {f: open(os.path.join(gdir, f)).read() for f in sorted(os.listdir(gdir)) if f.endswith((".c", ".cc", ".cpp", ".h"))}
    text = "\n".join(sources.values())
    called = set(re.findall(r"\b(iree_hal_thip_\w+)\s*\(", text))
    defined = set(re.findall(r"^(?:static |IREE_API_EXPORT )?[\w\*]+[ \*]+(iree_hal_thip_\w+)\([^;{]*\)\s*\{", text, re.M))
    undefined = {n for n in called - defined if not n.endswith("_t")}
    assert not undefined, sorted(undefined)
    readme = open(os.path.join(gdir, "README.md")).read()
    listed = set(re.findall(r"^\| `(iree_hal_torq_\w+)` \|", readme, re.M))
    used = {n for n in re.findall(r"\b(iree_hal_torq_\w+)\(", text) if not n.endswith("_t")}
    assert used == listed, sorted(used ^ listed)
    # the hunks for the reference's own files call only what the glue defines
    patch = open(os.path.join(gdir, "reference_hunks.patch")).read()
    hunks = set(re.findall(r"^\+.*?\b(iree_hal_thip_\w+)\s*\(", patch, re.M))
    assert hunks and hunks <= defined, sorted(hunks - defined)
    assert "IREE_HAL_THIP_EXECUTABLE_FORMAT" in sources["thip_native_executable.h"] and "IREE_HAL_THIP_EXECUTABLE_FORMAT" in patch

    abi = set(re.findall(r"\b(thip_[a-z_0-9]+)\s*\(", text))
    abi = {n for n in abi if not n.endswith("_t")}
    exported = set(runtime.EXPORTED_SYMBOLS)
    assert abi <= exported, sorted(abi - exported)


def test_reference_hunks_apply(tmp_path):
    """iree_glue/reference_hunks.patch against the reference checkout, where there is one (a dry run on copies)."""
    import shutil
    import subprocess
    ref = "/root/reference/runtime/driver"
    if not os.path.isdir(ref) or not shutil.which("patch"):
        pytest.skip("no reference checkout (or no patch tool) on this machine")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    dst = tmp_path / "runtime" / "driver"
    dst.mkdir(parents=True)
    for name in ("nop_executable_cache.cc", "torq_command_buffer.c"):
        shutil.copy(os.path.join(ref, name), dst / name)
    run = subprocess.run(["patch", "-p1", "--dry-run", "-i", os.path.join(root, "iree_glue", "reference_hunks.patch")], cwd=tmp_path,
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert run.returncode == 0 and "FAILED" not in run.stdout and "fuzz" not in run.stdout, run.stdout
