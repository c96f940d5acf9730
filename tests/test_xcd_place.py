"""The placement of one-dimensional grids on the eight XCDs (xcd_place in w2a8_common.h), checked on the host: the
function itself is compiled for the CPU and run over every small (sets, members) pair."""
import os
import shutil
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "slimkernels_amd", "csrc")

PROGRAM = r"""
#include "w2a8_common.h"
#include <cstdio>
#include <vector>
int main() {
    for (int sets = 1; sets <= 130; ++sets)
        for (int members = 1; members <= 16; ++members) {
            const int grid = w2a8::xcd_grid(sets, members);
            if (grid % 8 || grid < sets * members || grid >= sets * members + 8) { std::printf("grid %d %d\n", sets, members); return 1; }
            std::vector<int> seen(sets * members, 0), per_xcd(8, 0), home(sets, -1);
            int placed = 0, strays = 0;
            for (int wg = 0; wg < grid; ++wg) {
                int set = -1, member = -1;
                if (!w2a8::xcd_place(wg, sets, members, set, member)) continue;
                if (set < 0 || set >= sets || member < 0 || member >= members || seen[set * members + member]++) {
                    std::printf("bad place %d %d wg %d -> %d %d\n", sets, members, wg, set, member);
                    return 1;
                }
                ++placed;
                ++per_xcd[wg & 7];
                if (set < sets / 8 * 8) {   // a set dealt out whole: all members on one XCD, on consecutive places of its queue
                    if (home[set] < 0) home[set] = wg & 7;
                    if (home[set] != (wg & 7)) ++strays;
                    if (member > 0) {
                        int s2, m2;
                        if (!w2a8::xcd_place(wg - 8, sets, members, s2, m2) || s2 != set || m2 != member - 1) ++strays;
                    }
                }
            }
            int lo = per_xcd[0], hi = per_xcd[0];
            for (int x : per_xcd) { lo = x < lo ? x : lo; hi = x > hi ? x : hi; }
            if (placed != sets * members || hi - lo > 1 || strays) {
                std::printf("sets %d members %d: placed %d, per XCD %d..%d, strays %d\n", sets, members, placed, lo, hi, strays);
                return 1;
            }
        }
    std::printf("ok\n");
    return 0;
}
"""


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc to compile the header for the host")
def test_every_workgroup_placed_once_and_xcds_level(tmp_path):
    """Every (set, member) gets exactly one workgroup, no XCD holds more than one workgroup more than another, and the
    members of a set dealt out whole sit on consecutive places of one XCD's queue."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    src = tmp_path / "place.hip"
    src.write_text(PROGRAM)
    exe = tmp_path / "place"
    subprocess.run([hipcc, "--cuda-host-only", "-O1", "-std=c++17", "-I", CSRC, str(src), "-o", str(exe)], check=True,
                   capture_output=True, timeout=300)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and run.stdout.strip() == "ok", run.stdout + run.stderr
