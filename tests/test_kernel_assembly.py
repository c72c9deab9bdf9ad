"""The tiled prefill attention and the tiled and wide matrix products read their operands from
LDS by inline assembly and wait for them themselves.  The compiler's assembly of every variant
is checked for instructions that touch
a register between the read that fills it and the wait that covers it (`assembly_reads.py`),
and the check itself is pinned on two hand-written fragments.  Runs where hipcc is found."""

import os
import shutil
import subprocess

import pytest

import assembly_reads

CLEAN = """
_Z4testv:
\ts_load_dword s0, s[4:5], 0x0
.LBB0_1:
\t;;#ASMSTART
\tds_read_b128 v[4:7], v1
\t;;#ASMEND
\t;;#ASMSTART
\tds_read_b64_tr_b16 v[8:9], v2
\t;;#ASMEND
\t;;#ASMSTART
\ts_waitcnt lgkmcnt(1)
\t;;#ASMEND
\tv_mfma_f32_32x32x16_bf16 v[16:31], v[4:7], v[10:13], 0
\ts_cbranch_scc1 .LBB0_3
\tv_add_f32_e32 v3, v3, v16
.LBB0_3:
\t;;#ASMSTART
\ts_waitcnt lgkmcnt(0)
\t;;#ASMEND
\tv_mov_b32_e32 v14, v8
\ts_cbranch_scc0 .LBB0_1
\ts_endpgm
.Lfunc_end0:
"""


def test_the_check_tells_a_copy_before_the_wait_from_one_behind_it():
    assert assembly_reads.registers_touched_in_flight(CLEAN, "_Z4test") == {"_Z4testv": []}
    early = CLEAN.replace("\tv_add_f32_e32 v3, v3, v16\n", "\tv_mov_b32_e32 v15, v9\n")
    found = assembly_reads.registers_touched_in_flight(early, "_Z4test")["_Z4testv"]
    assert found == [("v_mov_b32_e32 v15, v9", [9])]
    # a register that is overwritten while its read is on its way, on one of two paths only
    clobber = CLEAN.replace("\tv_add_f32_e32 v3, v3, v16\n", "\tv_mov_b32_e32 v8, 0\n")
    assert assembly_reads.registers_touched_in_flight(clobber, "_Z4test")["_Z4testv"] == [("v_mov_b32_e32 v8, 0", [8])]
    # the compiler's own reads (outside the marks) are its own business
    own = CLEAN.replace("\t;;#ASMSTART\n\tds_read_b64_tr_b16 v[8:9], v2\n\t;;#ASMEND\n", "\tds_read_b64_tr_b16 v[8:9], v2\n")
    own = own.replace("\tv_add_f32_e32 v3, v3, v16\n", "\tv_mov_b32_e32 v15, v9\n")
    assert assembly_reads.registers_touched_in_flight(own, "_Z4test") == {"_Z4testv": []}


@pytest.mark.parametrize("name,prefix,least", [
    ("attention_prefill.hip", "_Z24attention_prefill_kernel", 30),   # every head size in its arrangements of waves
    ("attention_mixed.hip", "_Z22attention_mixed_kernel", 8),         # four head sizes x two kinds of loads
    ("gemm_tiled_bf16.hip", "_Z25gemm_nt_bf16_tiled_kernel", 60),    # tile shapes x ring depths x outputs x epilogues
    ("gemm_wide_bf16.hip", "_Z24gemm_nt_bf16_wide_kernel", 16),
])
def test_no_kernel_touches_a_register_in_flight(tmp_path, name, prefix, least):
    """The sources that read LDS by assembly, compiled to assembly with the library's own
    flags: no variant of their kernels names a register between its read and its wait."""
    from pagedserve_amd.ops import library

    hipcc = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc was not found")
    output = os.path.join(str(tmp_path), name.replace(".hip", ".s"))
    command = ([hipcc] + library.HIPCC_FLAGS + library.EXTRA_FLAGS.get(name, [])
               + ["-I", library.SOURCE_DIR, "-S", "--cuda-device-only",
                  os.path.join(library.SOURCE_DIR, name), "-o", output])
    done = subprocess.run(command, capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-2000:]
    with open(output) as handle:
        found = assembly_reads.registers_touched_in_flight(handle.read(), prefix)
    assert len(found) >= least, sorted(found)
    dirty = {kernel: problems[:3] for kernel, problems in found.items() if problems}
    assert not dirty, dirty
