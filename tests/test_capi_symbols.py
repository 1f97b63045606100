"""The shared library loads and exports every entry point include/rlt_rocm.h declares (no compute calls: runs without a GPU),
and the ctypes structure mirrors have the sizes the C compiler gives the header's structs."""
import ctypes as C
import os
import re
import subprocess
import tempfile

import helpers


def declared_symbols():
    text = open(os.path.join(helpers.ROOT, "include", "rlt_rocm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rlt_rocm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = helpers.package().load_library()
    names = declared_symbols()
    assert len(names) >= 50
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_library_has_no_oracle_dependency():
    path = helpers.package().capi.LIB_PATH
    out = subprocess.run(["ldd", path], capture_output=True, text=True).stdout
    assert "oracle" not in out
    src = os.path.join(helpers.ROOT, "rl-tools_amd")
    for dirpath, _, files in os.walk(src):
        for f in files:
            if f.endswith((".hip", ".h", ".py")):
                assert "oracle" not in open(os.path.join(dirpath, f)).read().lower() or f == "capi.py", (dirpath, f)


def test_structure_sizes_match_the_header():
    capi = helpers.capi
    # every struct the header declares (the opaque device handle aside) against its ctypes mirror: rlt_foo_bar <-> capi.FooBar
    text = open(os.path.join(helpers.ROOT, "include", "rlt_rocm.h")).read()
    declared = [n for n in re.findall(r"^typedef struct (rlt_[a-z0-9_]+)", text, flags=re.M) if n not in ("rlt_rocm_device", "rlt_rocm_graph")]      # the opaque handles
    assert len(declared) >= 26
    names = {n: getattr(capi, "".join(part.capitalize() for part in n[4:].split("_"))) for n in declared}
    prog = '#include <stdio.h>\n#include "rlt_rocm.h"\nint main(){' + "".join(f'printf("{n} %zu\\n", sizeof({n}));' for n in names) + "return 0;}"
    with tempfile.TemporaryDirectory() as d:
        open(os.path.join(d, "s.c"), "w").write(prog)
        subprocess.run(["gcc", "-I", os.path.join(helpers.ROOT, "include"), os.path.join(d, "s.c"), "-o", os.path.join(d, "s")], check=True)
        out = subprocess.run([os.path.join(d, "s")], capture_output=True, text=True, check=True).stdout
    for line in out.strip().splitlines():
        n, size = line.split()
        assert C.sizeof(names[n]) == int(size), (n, C.sizeof(names[n]), size)
