"""Bank model of the LDS access patterns the kernels are built on (the reference checks its shared-memory layouts
for bank conflicts with a probe kernel, slimkernels/cute/gemm/test_bc.cu; here the patterns are simple enough to
count on the host, and the rocprofv3 SQ_LDS_BANK_CONFLICT figures in profiles/ are the measured side).

Model: 64 banks of 4 bytes.  A 4-byte access of a wave is served in one pass when its 64 lanes hit 64 different
banks (same address = broadcast); a 16-byte access is served 16 lanes at a time, four consecutive banks per lane."""
import numpy as np


def conflict_degree(dword_addr, width_dwords):
    """Worst number of different addresses that fall on one bank within a pass."""
    dword_addr = np.asarray(dword_addr)
    lanes_per_pass = 64 // width_dwords
    worst = 1
    for p0 in range(0, 64, lanes_per_pass):
        per_bank = {}
        for a in dword_addr[p0:p0 + lanes_per_pass]:
            for d in range(width_dwords):
                per_bank.setdefault((a + d) % 64, set()).add(a + d)
        worst = max(worst, max(len(v) for v in per_bank.values()))
    return worst


LANE = np.arange(64)
COL, QUAD = LANE & 15, LANE >> 4


def test_operand_fragments_are_conflict_free():
    # a 1 KiB fragment (16 rows x 64 k, or a weight unit) lies in MFMA operand order: lane l's 16 bytes at 16 * l;
    # LDS-direct loads write it that way and every ds_read_b128 of the tiled and the 33..256-row kernel reads it so
    assert conflict_degree(LANE * 4, 4) == 1


def test_output_turn_of_the_tiled_and_the_mid_kernel():
    # the epilogues turn a 16 x 64 fp32 tile from accumulator order into rows through LDS with a row pitch of 68 floats
    pitch = 68
    for pp in range(4):
        for j in range(4):   # lane (col, quad) writes row quad * 4 + j, channel pp * 16 + col: the four quads 16 banks apart
            assert conflict_degree((QUAD * 4 + j) * pitch + pp * 16 + COL, 1) == 1
    for i in range(4):       # and reads back row i * 4 + quad, channels col * 4 .. + 3 as 16 bytes
        assert conflict_degree((i * 4 + QUAD) * pitch + COL * 4, 4) == 1
    # the same turn with a pitch of 64 or 65 floats would not do: the four quads of a write collide, or rows are not 16-byte aligned
    assert conflict_degree((QUAD * 4) * 64 + COL, 1) == 4
    assert ((np.arange(16) * 65) % 4 != 0).any()


def test_reduction_tile_of_the_skinny_kernels():
    # k-parts meet in red[wave][16][64 + 1] floats: lane (col, quad) writes row quad * 4 + j, column pp * 16 + col
    # (once per workgroup, 16 writes per lane: the quads land 4 banks apart, so a write pass is four-way conflicted; a
    # pitch of 68 would make it conflict-free at 3 KiB more LDS per workgroup - not worth it for ~50 cycles per workgroup)
    pitch = 65
    for pp in range(4):
        for j in range(4):
            assert conflict_degree((QUAD * 4 + j) * pitch + pp * 16 + COL, 1) == 4
    # and thread e reads element e of the tile (row e >> 6, column e & 63): consecutive lanes, consecutive banks
    e = LANE
    assert conflict_degree((e >> 6) * pitch + (e & 63), 1) == 1
