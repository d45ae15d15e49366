"""The host model of the kernels' walks (tests/host_model/walk_model.cpp), built with
AddressSanitizer and UndefinedBehaviorSanitizer and run on the CPU.

The model restates, without any device code, the work-item map and persistent
schedule of the dense forward kernel, its four-stage tile ring (and the five-stage ring of its short form) with the counted
vector-memory waits and barriers, the running-reference softmax, the window
form's block list and the dealing of decode chunks, and checks their invariants
over thousands of ragged shapes.  Each of its deliberate-mistake modes breaks one
of those protocols; the model has to notice every one of them.
"""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "host_model", "walk_model.cpp")

MISTAKES = {
    1: "the wait at the top of a tile leaves two tiles in flight",
    2: "the wait at the top of an item leaves tile 1 in flight",
    3: "a tile is requested into the stage of the tile before it",
    4: "no full wait and barrier before the last tiles of an item",
    5: "window list: the tail may start inside the sink blocks",
    6: "softmax: the reference point never moves",
    7: "odd rounds of the persistent schedule are reversed off by one",
    8: "the counted wait is used also behind partial output stores",
    9: "block-sparse: no barrier between the scores of tile 0 and the request of K of tile 2",
    10: "block-sparse: the list register behind the walked one is refilled with the wrong 64 entries",
    11: "short form: the wait at the top of an item always leaves one tile in flight",
    12: "short form: the wait at the top of a position leaves two tiles in flight",
    13: "window walk: a wave's positions are counted in keys, not in positions of the walk",
    14: "window walk: the sink tiles are not cut at the first tile of the band",
    15: "window walk: a tile at the window's lower edge is taken for unmasked",
}


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    exe = str(tmp_path_factory.mktemp("host_model") / "walk_model")
    subprocess.run(
        ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
         "-static-libasan", "-static-libubsan",  # the runtimes inside the executable: no library-order requirement
         "-fno-omit-frame-pointer", "-Wall", "-Wextra", "-Werror", SRC, "-o", exe],
        check=True, timeout=300)
    return exe


def _run(exe, *args):
    return subprocess.run([exe, *args], capture_output=True, text=True, timeout=300)


def test_walks_hold_their_invariants(model):
    r = _run(model)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "host model ok" in r.stdout
    for part in ("dense walk", "block-sparse walk", "softmax reference point", "decode lists and chunks", "window walk"):
        assert part in r.stdout


@pytest.mark.parametrize("mistake", sorted(MISTAKES), ids=lambda m: "mistake%d" % m)
def test_model_notices_a_broken_protocol(model, mistake):
    r = _run(model, str(mistake))
    assert r.returncode == 1, "not noticed: %s\n%s" % (MISTAKES[mistake], r.stdout[-2000:] + r.stderr[-2000:])
    assert "FAIL" in r.stdout
    assert "ERROR: AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr
