"""The loads that go from global memory straight into LDS are inline assembly, where the compiler's hazard handling
does not reach: a scalar register written by a vector instruction (v_readlane restoring a spilled scalar, for one)
must not be read by a memory instruction within five wait states.  This test emits the device assembly of the two
sources that contain such loads and scans every assembly block for that pattern (about a minute of compilation)."""
import os
import tempfile
from concurrent.futures import ThreadPoolExecutor

from spion_amd import build


def test_scanner_flags_a_restored_scalar_read_too_early():
    bad = """
_Zkernel:
	v_readlane_b32 s79, v184, 9
	;;#ASMSTART
	s_mov_b32 m0, s38
	s_nop 0
	buffer_load_dwordx4 v144, s[76:79], s82 offen lds
	;;#ASMEND
"""
    blocks, found = build.scan_sgpr_hazards(bad)
    assert blocks == 1 and len(found) == 1 and "s[76:79]" in found[0]
    blocks, found = build.scan_sgpr_hazards(bad.replace("s_nop 0", "s_nop 3"))
    assert blocks == 1 and found == []
    # a scalar written by scalar arithmetic is no such case
    blocks, found = build.scan_sgpr_hazards(bad.replace("v_readlane_b32 s79, v184, 9", "s_add_i32 s79, s1, s2"))
    assert found == []


def test_no_assembly_block_reads_a_vector_written_scalar_too_early():
    with tempfile.TemporaryDirectory() as tmp:
        srcs = ["sparse_attn.hip", "dense_attn.hip"]
        with ThreadPoolExecutor(max_workers=2) as ex:
            outs = list(ex.map(lambda s: build.emit_device_asm(s, os.path.join(tmp, s + ".s")), srcs))
        for src, out in zip(srcs, outs):
            blocks, found = build.scan_sgpr_hazards(open(out).read())
            assert blocks > 100, (src, blocks)  # the loads into LDS are there and were seen
            assert not found, f"{src}: {len(found)} sites, first: {found[0]}"
