"""The header tree as a drop-in: every public header name of the mirrored API exists under
include/thrust, every header that provides something compiles on its own with g++ (host pass:
the device system's calls are declarations there), and a header for something that is not
provided stops the build with a message instead of letting another Thrust installation on the
compiler's include path answer for it.

tests/golden/public_headers.txt is the list of names (thrust/*.h and its iterator, mr, system,
type_traits, async and random folders), one a line; it holds no source text.
"""
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
INCLUDE = os.path.join(HERE, "..", "include")
THRUST = os.path.join(INCLUDE, "thrust")


def _public_names():
    with open(os.path.join(HERE, "golden", "public_headers.txt")) as f:
        return [line.strip() for line in f if line.strip()]


def _provides(path):
    with open(path) as f:
        return "\n#error" not in f.read()


def _syntax_only(name):
    src = "#include <thrust/%s>\n#include <thrust/%s>\nint main() { return 0; }\n" % (name, name)
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I", INCLUDE, "-x", "c++", "-"], input=src,
                       capture_output=True, text=True)
    return name, r.returncode, r.stderr


def test_every_public_header_name_exists():
    missing = [n for n in _public_names() if not os.path.exists(os.path.join(THRUST, n))]
    assert missing == []


def test_every_providing_header_compiles_on_its_own():
    names = []
    for root, _, files in os.walk(THRUST):
        rel = os.path.relpath(root, THRUST)
        if rel.startswith(os.path.join("system", "hip")) or rel == os.path.join("iterator", "detail"):
            continue  # parts of other headers: kernels and their launchers, included where hipcc compiles
        for f in files:
            if f.endswith(".h") and _provides(os.path.join(root, f)):
                names.append(os.path.normpath(os.path.join(rel, f)))
    assert len(names) > 80
    with ThreadPoolExecutor(max_workers=8) as pool:
        results = list(pool.map(_syntax_only, sorted(names)))
    failed = ["%s: %s" % (n, err.strip().splitlines()[0] if err.strip() else rc) for n, rc, err in results if rc != 0]
    assert failed == []


def test_a_header_for_something_not_provided_stops_the_build():
    stubs = [n for n in _public_names() if not _provides(os.path.join(THRUST, n))]
    assert "complex.h" in stubs and os.path.join("system", "cuda", "execution_policy.h") in stubs
    for name in ("complex.h", "optional.h", os.path.join("system", "omp", "vector.h")):
        _, rc, err = _syntax_only(name)
        assert rc != 0 and "not provide" in err
