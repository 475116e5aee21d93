"""The chain engine's build products: one code object per HIP source and the kernarg table that lets the engine lay
out a dispatch's arguments itself.  The table comes from each code object's own metadata (guffin_amd/build.py
`kernarg_rows`, which refuses a kernel whose implicit arguments the engine does not fill); here: every code object
is there, every kernel has a row, and the implicit block follows the explicit arguments where a kernel has one."""
import glob
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HSACO = os.path.join(ROOT, "guffin_amd", "hsaco")


def rows():
    out = {}
    for line in open(os.path.join(HSACO, "kernargs.txt")):
        name, explicit_end, hidden_start = line.split()
        out[name] = (int(explicit_end), int(hidden_start))
    return out


def test_every_device_source_has_a_code_object():
    assert os.path.isdir(HSACO), "build first: python -m guffin_amd.build"
    sources = sorted(os.path.splitext(os.path.basename(p))[0] for p in glob.glob(os.path.join(ROOT, "guffin_amd", "csrc", "*.hip")))
    built = sorted(os.path.splitext(os.path.basename(p))[0] for p in glob.glob(os.path.join(HSACO, "*.hsaco")))
    assert sources == built


def test_kernarg_table_covers_the_step_kernels():
    table = rows()
    assert len(table) >= 100
    for fragment in ("gateup_geglu_kernel", "gemv_packed_kernel", "gemv_packed_multi_kernel", "attn_partial_kernel",
                     "attn_merge_kernel", "rms_norm_add_norm_regs_kernel", "resident_blocks_kernel", "spec_accept_kernel",
                     "threshold_select_kernel", "commit_rows_kernel"):
        assert any(fragment in name for name in table), fragment
    for name, (explicit_end, hidden_start) in table.items():
        assert explicit_end >= 0
        assert hidden_start == -1 or hidden_start == (explicit_end + 7) // 8 * 8, name


def test_table_matches_the_code_objects_metadata():
    from guffin_amd import build
    table = rows()
    seen = 0
    for path in sorted(glob.glob(os.path.join(HSACO, "*.hsaco"))):
        for name, explicit_end, hidden_start in build.kernarg_rows(path):
            assert table[name] == (explicit_end, hidden_start)
            seen += 1
    assert seen == len(table)
