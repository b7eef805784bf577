"""The host build of the library's kernels and host side (tests/host_block/) under the address,
undefined-behaviour and thread sanitizers (GPU sanitizers do not exist on the target; host code is where
they run). tests/host_block/sanitize_main.cpp calls fta_plan / fta_decode on buffers of exactly their size
(contiguous and paged caches, ragged tiles, empty and over-long sequences, additive and packed masks; fp32
through the shuffle kernel, bf16 through the MFMA kernel in its 4-wave, 8-wave pipelined, head_dim 256 and
key-halves forms, with and without the merge inside the launch) and checks the results against a plain
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

import pytest

from flash_tree_attn_amd import build as fta_build

HERE = os.path.dirname(os.path.abspath(__file__))
CLANG = os.path.join(os.path.dirname(fta_build.HIPCC), "..", "llvm", "bin", "clang++")
SOURCES = ["fta_host.cpp", "stage1_shuffle.hip", "stage2_merge.hip", "append_kv.hip"]


@pytest.mark.parametrize("sanitize", ["address,undefined", "thread"])
def test_host_build_is_clean_under(sanitize, tmp_path):
    if not os.path.exists(CLANG):
        pytest.skip("no host clang++")
    flags = ["-x", "c++", "-std=c++20", "-O1", "-g", f"-fsanitize={sanitize}", "-fno-omit-frame-pointer", "-pthread",
             "-I", os.path.join(HERE, "host_block"), "-I", fta_build.INCLUDE, "-I", fta_build.CSRC]
    procs, objs = [], []
    for src in [os.path.join(fta_build.CSRC, s) for s in SOURCES] + [os.path.join(HERE, "host_block", n) for n in ("stage1_mfma_host.cpp", "sanitize_main.cpp")]:
        obj = str(tmp_path / (os.path.basename(src) + ".o"))
        # the MFMA kernel's twenty instantiations take minutes to optimise under a sanitizer and seconds not to
        level = ["-O0"] if src.endswith("stage1_mfma_host.cpp") else []
        procs.append(subprocess.Popen([CLANG, *flags, *level, "-c", src, "-o", obj], stdout=subprocess.PIPE, stderr=subprocess.STDOUT))
        objs.append(obj)
    for proc in procs:
        log = proc.communicate()[0]
        assert proc.returncode == 0, log.decode()[-3000:]
    exe = str(tmp_path / "sanitize_host")
    subprocess.run([CLANG, f"-fsanitize={sanitize}", "-pthread", *objs, "-o", exe], check=True, capture_output=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0", UBSAN_OPTIONS="halt_on_error=1", TSAN_OPTIONS="halt_on_error=0")
    # under the thread sanitizer the MFMA cases run twice: loads that land when issued, then loads that land as late as the waits allow
    r = subprocess.run([exe, "mfma"] + (["both"] if sanitize == "thread" else []), capture_output=True, text=True, timeout=900, env=env)
    text = r.stdout + r.stderr
    for sign in ("AddressSanitizer", "runtime error", "data race", "ThreadSanitizer", "FAILED"):
        assert sign not in text, text[-3000:]
    assert r.returncode == 0 and text.strip().endswith("clean"), text[-2000:]
    assert text.count("bf16/mfma") == (14 if sanitize == "thread" else 7), text[-2000:]
