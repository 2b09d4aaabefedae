"""The drop-in boundary as a C caller sees it (no GPU needed):
every function the public headers declare is exported by libcutt.so, the headers compile as
plain C99, and a C program linked against the library gets the documented error codes on the
paths that return before any device access."""
import ctypes
import os
import re
import subprocess

import cutt_amd

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
INCLUDE = os.path.join(ROOT, "include")


def declared_functions():
    names = set()
    for hdr in ("cutt.h", "cutt_ext.h"):
        text = open(os.path.join(INCLUDE, hdr)).read()
        text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)  # comments mention functions too
        for m in re.finditer(r"\b(cutt[A-Z]\w*)\s*\(", text):
            names.add(m.group(1))
    return sorted(names)


def test_every_declared_function_is_exported():
    names = declared_functions()
    for must in ("cuttPlan", "cuttPlanMeasure", "cuttExecute", "cuttDestroy", "cuttGetPlanInfo",
                 "cuttCandidatesCreate", "cuttModelShTransactions"):
        assert must in names
    lib = ctypes.CDLL(cutt_amd.lib_path())
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_plan_functions_have_c_linkage():
    # the dynamic symbol table holds the four plan functions under their plain C names
    out = subprocess.run(["nm", "-D", "--defined-only", cutt_amd.lib_path()], stdout=subprocess.PIPE, text=True,
                         check=True).stdout
    syms = {l.split()[-1] for l in out.splitlines() if l.strip()}
    for n in ("cuttPlan", "cuttPlanMeasure", "cuttExecute", "cuttDestroy"):
        assert n in syms


def test_headers_are_plain_c_and_a_c_caller_links(tmp_path):
    exe = str(tmp_path / "c_abi_check")
    libdir = os.path.dirname(cutt_amd.lib_path())
    cmd = ["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", INCLUDE,
           os.path.join(HERE, "c_abi_check.c"), "-o", exe, "-L", libdir, "-lcutt", "-Wl,-rpath," + libdir,
           "-Wl,-rpath-link,/opt/rocm/lib"]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode == 0, (r.returncode, r.stdout)
    assert "c abi ok" in r.stdout
