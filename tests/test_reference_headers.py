"""The hip extension's sources against nnabla's OWN headers.

In this repository the extension (``nnabla_amd/csrc/hip/*.cpp``, ``nnabla_amd/csrc/include/nbla/hip/**``) is built
against a from-scratch core that carries nbla's names.  A maintainer dropping it into nnabla compiles the same files
against nnabla's headers instead.  This test does exactly that, syntax only (``g++ -fsyntax-only`` with nnabla's
``include/`` first on the search path): every source and every extension header must compile, and every ``nbla/...``
header they pull in -- apart from the extension's own ``nbla/hip/...`` -- must resolve into nnabla's tree, not into
the look-alike core.  Nothing is copied, linked or run; the test is skipped where the nnabla checkout is absent."""
import glob
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "nnabla_amd", "csrc")
REF_INCLUDE = "/root/reference/include"

pytestmark = pytest.mark.skipif(
    not os.path.isdir(os.path.join(REF_INCLUDE, "nbla")) or shutil.which("g++") is None,
    reason="needs the nnabla checkout at /root/reference and g++")

FLAGS = ["g++", "-std=c++14", "-fsyntax-only", "-Wall", "-Wno-unused-function",
         "-I", REF_INCLUDE, "-I", os.path.join(CSRC, "include"), "-I", os.path.join(ROOT, "include")]

SOURCES = sorted(glob.glob(os.path.join(CSRC, "hip", "*.cpp")))
HEADERS = sorted(glob.glob(os.path.join(CSRC, "include", "nbla", "hip", "**", "*.hpp"), recursive=True))


def _compile(args, stdin=None):
    return subprocess.run(FLAGS + args, input=stdin, capture_output=True, text=True, timeout=300)


def test_the_file_lists_are_what_the_extension_consists_of():
    assert [os.path.basename(s) for s in SOURCES] == ["functions.cpp", "hip.cpp", "init.cpp", "shapes.cpp"]
    assert len(HEADERS) >= 10


@pytest.mark.parametrize("source", SOURCES, ids=[os.path.basename(s) for s in SOURCES])
def test_extension_source_compiles_against_nnabla_headers(source):
    r = _compile([source])
    assert r.returncode == 0 and "error" not in r.stderr, r.stderr[-4000:]


@pytest.mark.parametrize("header", HEADERS, ids=[os.path.relpath(h, os.path.join(CSRC, "include")) for h in HEADERS])
def test_extension_header_compiles_alone_against_nnabla_headers(header):
    rel = os.path.relpath(header, os.path.join(CSRC, "include"))
    r = _compile(["-x", "c++", "-"], stdin="#include <%s>\n" % rel)
    assert r.returncode == 0 and "error" not in r.stderr, r.stderr[-4000:]


@pytest.mark.parametrize("source", SOURCES, ids=[os.path.basename(s) for s in SOURCES])
def test_only_extension_headers_come_from_this_repository(source):
    """The dependency list of each source: nbla/hip/** and the C-ABI header from here, every other nbla header from
    nnabla's own include directory."""
    r = subprocess.run(FLAGS[:2] + ["-M"] + FLAGS[5:] + [source], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-4000:]
    deps = [d for d in r.stdout.replace("\\\n", " ").split()[1:] if "/nbla" in d]
    ours = [d for d in deps if os.path.abspath(d).startswith(ROOT)]
    theirs = [d for d in deps if os.path.abspath(d).startswith(REF_INCLUDE)]
    assert theirs, "no nnabla header was used at all"
    allowed = (os.path.join(CSRC, "include", "nbla", "hip") + os.sep, os.path.join(ROOT, "include") + os.sep,
               os.path.join(CSRC, "hip") + os.sep)
    stray = [d for d in ours if not os.path.abspath(d).startswith(allowed)]
    assert not stray, "resolved into the look-alike core instead of nnabla: %s" % stray
