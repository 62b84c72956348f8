"""Register budgets that are part of a kernel's design, held to the build's own resource report.

The 8-bit attention kernels' register budget is part of their design: one wave per SIMD with
the whole register file, 128 accumulators in ordinary registers, the q terms in the accumulation
registers (rivoli_amd/csrc/mla_attend_f8.hpp). A compiler or source change that makes them spill
still gives right answers, only several times slower, so the build's own resource report is held
to "no scratch memory" here. The scored block selection keeps a row's keys in registers and its
phases must not share per-element lane masks: 32 of them do not fit the scalar registers, and
when they spilled (to lanes of a vector register, a write and a read each) a quarter of the
kernel's vector instructions were spill traffic. Compiles one file per test; needs hipcc, no
GPU."""
import os
import re
import shutil
import subprocess

import pytest

from rivoli_amd import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which(build.hipcc()) is None, reason="hipcc not found")
def test_eight_bit_attention_kernels_do_not_spill(tmp_path):
    src = os.path.join(build.CSRC, "mla_attend.hip")
    cmd = [build.hipcc(), f"--offload-arch={build.offload_arch()}", "-O3", "-std=c++17", "-fPIC",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(ROOT, "include")] + build.EXTRA_FLAGS.get("mla_attend.hip", []) + \
          ["-Rpass-analysis=kernel-resource-usage", "-c", src, "-o", str(tmp_path / "m.o")]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    # remarks come in blocks: "Function Name: <mangled>" followed by that kernel's figures
    blocks = re.split(r"remark: Function Name: ", res.stderr)[1:]
    seen = 0
    for b in blocks:
        name = b.split()[0]
        if "mla_attend_paged_kernel" not in name or not name.endswith("Lb1EEEvNS_10AttendArgsE"):
            continue  # the last template argument (true) marks the 8-bit kernels
        seen += 1
        scratch = int(re.search(r"ScratchSize \[bytes/lane\]: (\d+)", b).group(1))
        occupancy = int(re.search(r"Occupancy \[waves/SIMD\]: (\d+)", b).group(1))
        lds = int(re.search(r"LDS Size \[bytes/block\]: (\d+)", b).group(1))
        assert scratch == 0, f"{name} spills {scratch} bytes per lane"
        assert occupancy == 1, name
        assert lds <= 160 * 1024, name
    assert seen == 4, f"expected the dense and row-list kernels of both 8-bit modes, saw {seen}"


def _resource_blocks(src_name):
    src = os.path.join(build.CSRC, src_name)
    cmd = [build.hipcc(), f"--offload-arch={build.offload_arch()}", "-O3", "-std=c++17", "-fPIC",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(ROOT, "include")] + build.EXTRA_FLAGS.get(src_name, []) + \
          ["-Rpass-analysis=kernel-resource-usage", "-c", src, "-o", os.devnull]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    return re.split(r"remark: Function Name: ", res.stderr)[1:]


@pytest.mark.skipif(shutil.which(build.hipcc()) is None, reason="hipcc not found")
def test_block_selection_keeps_its_masks_out_of_memory():
    seen = 0
    for b in _resource_blocks("index_topk.hip"):
        name = b.split()[0]
        if "block_select_bisect_kernel" not in name:
            continue
        seen += 1
        assert int(re.search(r"SGPRs Spill: (\d+)", b).group(1)) == 0, name
        assert int(re.search(r"VGPRs Spill: (\d+)", b).group(1)) == 0, name
        assert int(re.search(r"ScratchSize \[bytes/lane\]: (\d+)", b).group(1)) == 0, name
        assert int(re.search(r"Occupancy \[waves/SIMD\]: (\d+)", b).group(1)) == 8, name
    assert seen == 6, f"expected the six widths of the register form, saw {seen}"


@pytest.mark.skipif(shutil.which(build.hipcc()) is None, reason="hipcc not found")
def test_block_scorer_keeps_its_row_and_both_chunk_buffers_in_registers():
    """The block scorer holds a 128-value row per lane and two 32-value chunks of the query in
    scalar registers; a spill of either turns its two instructions per term into many."""
    seen = 0
    for b in _resource_blocks("block_index.hip"):
        name = b.split()[0]
        if "index_score_blocks_128" not in name:
            continue
        seen += 1
        if "split" not in name:   # the decode kernel is bound by latency, not by issue
            assert int(re.search(r"SGPRs Spill: (\d+)", b).group(1)) == 0, name
        assert int(re.search(r"VGPRs Spill: (\d+)", b).group(1)) == 0, name
        assert int(re.search(r"ScratchSize \[bytes/lane\]: (\d+)", b).group(1)) == 0, name
        assert int(re.search(r"Occupancy \[waves/SIMD\]: (\d+)", b).group(1)) >= 3, name
    assert seen == 2


def test_the_build_refuses_an_attention_object_that_spills():
    """build.check_resources is what build_kernels applies to mla_attend.hip's resource report:
    scratch memory or too much LDS in an 8-bit attention kernel raises instead of linking."""
    head = "x.hip:1:1: remark: Function Name: _ZN2rk23mla_attend_paged_kernelILi2ELi2ELi0ELb0ELb1EEEvNS_10AttendArgsE\n"
    fine = head + "    ScratchSize [bytes/lane]: 0\n    LDS Size [bytes/block]: 85632\n"
    build.check_resources("mla_attend.hip", fine)
    build.check_resources("kv_gather.hip", "")                        # other files are not held to it
    for bad in (fine.replace("lane]: 0", "lane]: 44"), fine.replace("85632", "170000"), ""):
        with pytest.raises(RuntimeError):
            build.check_resources("mla_attend.hip", bad)
