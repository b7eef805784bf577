"""The host build of the library's kernels and host side (tests/host_block/) under the address,
undefined-behaviour and thread sanitizers (GPU sanitizers do not exist on the target; host code is where
they run). tests/host_block/sanitize_main.cpp calls fta_plan / fta_decode on buffers of exactly their size
(contiguous and paged caches, ragged tiles, empty and over-long sequences, additive and packed masks; fp32
through the shuffle kernel, bf16 through the MFMA kernel in its 4-wave, 8-wave pipelined, head_dim 256 and
key-halves forms and as the 64-row-wave kernel with its assembly statements interpreted (tests/test_host_block_wide.py),
with and without the merge inside the launch) and checks the results against a plain
double-precision attention.
  * address / undefined: a read or write one element past a tensor, a page, the scratch, an LDS array (the
    MFMA kernel's LDS addresses are checked against the launch's LDS size by the stand-ins themselves);
  * thread: every GPU thread is a host thread here and the only synchronisation is what the kernels ask for
    (`__syncthreads`, the workgroup barrier, wave barriers, shuffles), so a missing barrier is a data race
    the sanitizer reports. A direct global->LDS load lands the moment it is issued here, the earliest it
    ever could, so a ring stage that is requested while another wave may still read it is a race too; in a second
    pass the loads land only when a vmcnt wait of their wave forces them to, the latest the hardware allows, so a
    stage that is read before its loading wave has waited and passed a barrier is a race as well.
    (Checked by hand: without the barrier in front of the ranking loop of item_by_order it reports 12 races,
    without the barrier of the MFMA kernel's synchronisation point 192.)"""
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from flash_tree_attn_amd import build as fta_build

HERE = os.path.dirname(os.path.abspath(__file__))
CLANG = os.path.join(os.path.dirname(fta_build.HIPCC), "..", "llvm", "bin", "clang++")
SOURCES = ["fta_host.cpp", "stage1_shuffle.hip", "stage2_merge.hip", "append_kv.hip"]


def test_host_build_is_clean_under_the_sanitizers(tmp_path):
    if not os.path.exists(CLANG):
        pytest.skip("no host clang++")
    from test_host_block_wide import build_host_library_with_wide
    kinds = ["address,undefined", "thread"]

    def build(sanitize):
        out = tmp_path / sanitize.split(",")[0]
        out.mkdir()
        return build_host_library_with_wide(str(out), extra_flags=["-g", f"-fsanitize={sanitize}", "-fno-omit-frame-pointer"], link_flags=[f"-fsanitize={sanitize}"],
                                            extra_sources=[os.path.join(HERE, "host_block", "sanitize_main.cpp")], output="sanitize_host", shared=False)

    with ThreadPoolExecutor(max_workers=2) as pool:      # both builds, then both runs, side by side
        exes = list(pool.map(build, kinds))
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0", UBSAN_OPTIONS="halt_on_error=1", TSAN_OPTIONS="halt_on_error=0")
    # under the thread sanitizer the MFMA cases run twice: loads that land when issued, then loads that land as late as the waits allow
    runs = [subprocess.Popen([exe, "mfma"] + (["both"] if sanitize == "thread" else []), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
            for exe, sanitize in zip(exes, kinds)]
    for run, sanitize in zip(runs, kinds):
        text = run.communicate(timeout=900)[0]
        for sign in ("AddressSanitizer", "runtime error", "data race", "ThreadSanitizer", "FAILED"):
            assert sign not in text, (sanitize, text[-3000:])
        assert run.returncode == 0 and text.strip().endswith("clean"), (sanitize, text[-2000:])
        assert text.count("bf16/mfma") == (18 if sanitize == "thread" else 9), (sanitize, text[-2000:])
