"""The C-ABI library loads and exports exactly what include/plr.h declares
(no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "plr.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(plr_[a-z_]+)\s*\(", text)))


def test_header_and_binding_agree():
    from paracel_amd import capi

    assert declared_symbols() == sorted(name for name, _, _ in capi.SYMBOLS)


def test_library_exports_every_declared_symbol():
    from paracel_amd import capi

    lib = ctypes.CDLL(capi.lib_path())
    for name in declared_symbols():
        assert hasattr(lib, name), name
    loaded = capi.load_library()
    assert loaded.plr_version().decode().startswith("plr ")
    assert loaded.plr_last_error(None) is not None


def test_header_is_plain_c99_and_a_c_caller_links(tmp_path):
    """include/plr.h is a C header: it compiles as C99 with -pedantic -Wall -Werror on its own,
    and the plain-C caller that binds it links against libplr.so (no C++ runtime needed by
    the caller)."""
    import subprocess

    from paracel_amd import capi

    probe = tmp_path / "probe.c"
    probe.write_text('#include "plr.h"\nint main(void) { return (int)PLR_OK; }\n')
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only",
                    "-I", os.path.join(ROOT, "include"), str(probe)], check=True)
    out = tmp_path / "plr_c_caller"
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror",
                    "-I", os.path.join(ROOT, "include"), "-o", str(out),
                    os.path.join(ROOT, "paracel_amd", "examples", "plr_c_caller.c"),
                    "-L", os.path.dirname(capi.lib_path()), "-lplr"], check=True)
    assert out.exists()


def test_product_does_not_touch_the_oracle():
    # the oracle is test infrastructure: nothing under paracel_amd/ or include/ may
    # import, link or load it
    bad = []
    for base in ("paracel_amd", "include"):
        for dp, _, files in os.walk(os.path.join(ROOT, base)):
            for f in files:
                if f.endswith((".py", ".hip", ".hpp", ".h", ".c", ".cpp")):
                    if "oracle" in open(os.path.join(dp, f), errors="ignore").read():
                        bad.append(os.path.join(dp, f))
    assert not bad, bad


def test_no_silent_cpu_path_without_a_gpu():
    """Without a usable GPU the library must refuse to create a context (loudly, with a
    message) -- there is no CPU fallback to fall into.  On a GPU box this test checks the
    out-of-range device id instead."""
    import pytest

    from paracel_amd import Plr, PlrError

    try:
        import torch

        have_gpu = torch.cuda.device_count() > 0
    except Exception:  # torch is only used to count devices without initialising HIP here
        have_gpu = os.path.exists("/dev/kfd")
    with pytest.raises(PlrError) as e:
        Plr(4096 if have_gpu else 0)
    assert e.value.code in (-1, -2) and len(str(e.value)) > 20
