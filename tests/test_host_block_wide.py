"""The 64-row-wave kernel, whole, on host threads: the product's C++ around the assembly statements
(stage1_mfma_kernel.h, MODE == kWide, compiled for the host as in tests/test_host_block_mfma.py) AND the statements
themselves, interpreted from the text that gen_wide_loop.py renders into wide_loop_asm.inc
(tests/host_block/gfx950_asm_host.h: every host thread is one lane with its own registers; matrix products, the
half-wave swap, the transposing LDS read and vector compares meet in the wave's exchange area). The rendering of
the statements as interpreter calls is made here from the generator's own output, whose equality with the committed
file tests/test_kernel_asm.py asserts.

This is the kernel the library only runs when asked (force_kernel = FTA_KERNEL_MFMA_WIDE). What the run pins: the
hand-over between the C++ and the statements (ring offsets, tile counts, the address of the next tile, what comes
back), the tree block and the ragged tail through the masked halves, the loop with its exact redo when a row maximum
rises late, the ring protocol between the four waves, under both models of the global->LDS loads and with LDS reads
that deliver only at their lgkmcnt wait; a vector instruction that names a register of a read still in flight, or a
register the operand lists do not bind (all start as NaN patterns), fails the run. Not shown: issue hazards and the
compiler's registers around the statements (gen_wide_loop.py: hazards(), verify(); tests/test_kernel_asm.py), speed.

TEST INFRASTRUCTURE ONLY: nothing under flash_tree_attn_amd/ knows of this build."""
import ctypes as C
import importlib.util
import os
import re
import subprocess

import pytest
import torch

from flash_tree_attn_amd import _lib
from flash_tree_attn_amd import build as fta_build
from test_host_block_kernels import CLANG, HERE, SOURCES, TOL, HostCall, make, oracle
from test_zz_stage_entries_gpu import expected_partials, live_splits

WIDE, MFMA = _lib.KERNEL_MFMA_WIDE, _lib.KERNEL_MFMA


def _generator():
    spec = importlib.util.spec_from_file_location("gen_wide_loop", os.path.join(fta_build.CSRC, "gen_wide_loop.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def statements_as_interpreter_calls() -> str:
    """Every macro of wide_loop_asm.inc with the same instruction text, as a call of host_asm::run with the operand
    lists turned into (register, object, written back) bindings."""
    gen = _generator()

    def statement(name, body, ops, bf16):
        binds = [f'{{"{m.group(2)}", host_asm::bits({m.group(3)}), {"true" if m.group(1) else "false"}}}'
                 for m in re.finditer(r'"(\+?)\{(\w+)\}"\(([^)]+)\)', ops)]
        assert len(binds) == ops.count("{"), name
        lines = [f"#define {name}() do {{ \\", "    static const host_asm::Program prog_( \\"]
        lines += [f'      "{ins}\\n" \\' for ins in body]
        lines += ["    ); \\", "    const host_asm::Binding bind_[] = { \\"]
        lines += [f"      {b}, \\" for b in binds]
        lines += ["    }; \\", f"    host_asm::run(prog_, bind_, sizeof(bind_) / sizeof(bind_[0]), {'true' if bf16 else 'false'}); \\", "  } while (0)"]
        return lines

    out = []
    for D in (128, 64):
        for dtype in ("bf16", "f16"):
            out += statement(f"FTA_WIDE_LOOP_{D}_{dtype.upper()}", gen.gen(D, dtype), gen.operands(D), dtype == "bf16")
            for H in (0, 1):
                out += statement(f"FTA_WIDE_MASKED_{D}_{dtype.upper()}_H{H}", gen.gen_masked(D, dtype, H), gen.operands_masked(D), dtype == "bf16")
    return "\n".join(out) + "\n"


def build_host_library_with_wide(out_dir, extra_flags=(), link_flags=(), extra_sources=(), output="libfta_host_wide.so", shared=True):
    """Compiles the product sources and both MFMA host units into `out_dir`; returns the path of the result."""
    with open(os.path.join(out_dir, "wide_loop_host.inc"), "w") as f:
        f.write(statements_as_interpreter_calls())
    flags = ["-x", "c++", "-std=c++20", "-O1", "-fPIC", "-pthread", *extra_flags, "-I", str(out_dir), "-I", os.path.join(HERE, "host_block"),
             "-I", fta_build.INCLUDE, "-I", fta_build.CSRC, "-DFTA_HOST_WITH_WIDE_UNIT", '-DFTA_HOST_WIDE_LOOP_INC="wide_loop_host.inc"']
    srcs = [os.path.join(fta_build.CSRC, s) for s in SOURCES] + [os.path.join(HERE, "host_block", n) for n in ("stage1_mfma_host.cpp", "stage1_mfma_wide_host.cpp")] + list(extra_sources)
    procs, objs = [], []
    for src in srcs:
        obj = os.path.join(out_dir, os.path.basename(src) + ".o")
        level = ["-O0"] if "stage1_mfma" in os.path.basename(src) else []     # many instantiations: seconds instead of minutes
        procs.append(subprocess.Popen([CLANG, *flags, *level, "-c", src, "-o", obj], stdout=subprocess.PIPE, stderr=subprocess.STDOUT))
        objs.append(obj)
    for proc in procs:
        log = proc.communicate()[0]
        assert proc.returncode == 0, log.decode()[-3000:]
    path = os.path.join(out_dir, output)
    subprocess.run([CLANG, *(["-shared"] if shared else []), "-pthread", *link_flags, *objs, "-o", path], check=True, capture_output=True)
    return path


@pytest.fixture(scope="module")
def host_lib(tmp_path_factory):
    if not os.path.exists(CLANG):
        pytest.skip("no host clang++")
    lib = C.CDLL(build_host_library_with_wide(str(tmp_path_factory.mktemp("host_block_wide"))))
    for name in ("fta_decode", "fta_decode_stage1", "fta_decode_stage2"):
        getattr(lib, name).argtypes = [C.POINTER(_lib.FtaArgs), C.c_void_p]
    lib.fta_plan.argtypes = [C.POINTER(_lib.FtaArgs), C.c_int, C.POINTER(_lib.FtaPlanOut)]
    lib.host_block_loads_land_late.argtypes = [C.c_int]
    assert lib.fta_abi_version() == _lib.ABI_VERSION
    return lib


@pytest.fixture(autouse=True)
def loads_land_when_issued(host_lib):
    host_lib.host_block_loads_land_late(0)
    yield
    host_lib.host_block_loads_land_late(0)


CASES = [
    # name                                       bsz hq hkv  L   D    T    lens            splits dtype         hot   late
    ("6 full tiles", 1, 4, 1, 64, 128, 384, [384], 1, torch.bfloat16, None, False),
    ("1 .. 4 full tiles, loads land late", 4, 4, 1, 64, 128, 256, [64, 128, 192, 256], 1, torch.bfloat16, None, True),
    ("ragged tails, an empty cache", 4, 4, 1, 64, 128, 512, [500, 150, 37, 0], 1, torch.bfloat16, None, False),
    ("3 splits, loads land late", 1, 4, 1, 64, 128, 640, [640], 3, torch.bfloat16, None, True),
    ("192 rows: one wave without rows", 1, 6, 1, 32, 128, 320, [300], 2, torch.bfloat16, None, False),
    ("160 rows of 16", 1, 10, 1, 16, 128, 256, [256], 1, torch.bfloat16, None, False),
    ("a late key raises every row maximum", 1, 4, 1, 64, 128, 512, [512], 1, torch.bfloat16, 400, False),
    ("fp16, late key, loads land late", 1, 4, 1, 64, 128, 384, [384], 1, torch.float16, 300, True),
    ("head_dim 64", 1, 4, 1, 64, 64, 384, [330], 2, torch.bfloat16, None, False),
    ("head_dim 64, fp16, late key", 1, 8, 1, 32, 64, 384, [384], 1, torch.float16, 250, False),
    ("a tree of 70 tokens: two tree tiles", 1, 2, 1, 70, 128, 192, [130], 1, torch.bfloat16, None, False),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: c[0])
def test_64_row_wave_kernel_on_host_threads(host_lib, case):
    name, bsz, hq, hkv, L, D, T, lens, splits, dtype, hot, late = case
    x = make(75, bsz, hq, hkv, L, D, T, dtype, lens)
    if hot is not None:      # one key far along the stream that every row of the first head group scores highest
        x["k_cache"][:, :, hot, :] = (x["q"][:, :: hq // hkv, 0, :].float() * 3).to(dtype)
    ref = oracle(x)
    call = HostCall(host_lib, x, splits=splits, kernel=WIDE)
    assert call.plan.kernel == MFMA and call.plan.rows_per_wg == 256 and call.plan.mfma_loop == 1
    host_lib.host_block_loads_land_late(1 if late else 0)
    out = call.run().clone()
    assert torch.isfinite(out).all()
    torch.testing.assert_close(out.float(), ref, **TOL[dtype])
    host_lib.host_block_loads_land_late(0)
    if hot is not None or bsz == 1 and splits == 1:      # next to the 8-wave loop it stands in for (a few cases: that kernel has its own tests)
        narrow = HostCall(host_lib, x, splits=splits, kernel=MFMA)
        assert narrow.plan.mfma_loop == 0
        torch.testing.assert_close(out.float(), narrow.run().float(), **TOL[dtype])


# Keys of more spread than N(0, 1): a few keys carry each row. The loop's lazy softmax exponentiates against a stale
# reference, so every probability of a row, its largest included, is rounded to bf16 (2^-9 relative) where the other
# loops hold the largest exactly at 1, and full tiles take no compensating product with the rounding residue (the
# 8-wave, 4-wave and key-halves loops do: tests/test_host_block_mfma_forms.py). At twice the spread the loop stays inside
# the tolerance; at four times it does not (1.06 - 1.42 of atol 2e-3 / rtol 1e-2 here, 3 of 32768 values beyond it
# on the GPU at 1024 keys). That is a known limit of this opt-in loop: the rows stay here, marked, until it is lifted.
@pytest.mark.parametrize("scale_k,seed,keys", [
    (2.0, 0, 512), (2.0, 3, 512), (2.0, 75, 1024),
    pytest.param(4.0, 0, 512, marks=pytest.mark.xfail(strict=True, reason="known limit: bf16 probabilities of peaked rows, no residue product in the assembly loop")),
    pytest.param(4.0, 3, 512, marks=pytest.mark.xfail(strict=True, reason="known limit: bf16 probabilities of peaked rows, no residue product in the assembly loop")),
])
def test_64_row_wave_kernel_on_peaked_rows(host_lib, scale_k, seed, keys):
    x = make(seed, 1, 4, 1, 64, 128, keys, torch.bfloat16, [keys])
    x["k_cache"] = (x["k_cache"].float() * scale_k).to(torch.bfloat16)
    call = HostCall(host_lib, x, splits=1, kernel=WIDE)
    assert call.plan.mfma_loop == 1
    torch.testing.assert_close(call.run().float(), oracle(x), **TOL[torch.bfloat16])


def test_64_row_wave_kernel_partials_and_merge_inside_the_launch(host_lib):
    lens, tmax, S = [330, 0], 2048, 3
    x = make(77, 2, 3, 1, 64, 128, tmax, torch.bfloat16, lens)
    call = HostCall(host_lib, x, splits=S, kernel=WIDE)
    chunk = call.plan.chunk_for(max(lens))
    assert call.plan.num_splits == S and chunk < call.plan.chunk
    call.run("fta_decode_stage1")
    for b, t_b in enumerate(lens):
        parts = expected_partials(x, b, chunk, S)
        assert len(parts) == live_splits(t_b, chunk, S)
        for s, (o_ref, lse_ref) in enumerate(parts):
            torch.testing.assert_close(call.lse[b, :, s], lse_ref, atol=2e-3, rtol=1e-3)
            torch.testing.assert_close(call.mid[b, :, s], o_ref, **TOL[torch.bfloat16])
        for s in range(len(parts), S):
            assert torch.isnan(call.mid[b, :, s]).all() and torch.isnan(call.lse[b, :, s]).all()
    ref = call.run("fta_decode_stage2").clone()
    torch.testing.assert_close(ref.float(), oracle(x), **TOL[torch.bfloat16])
    fused = HostCall(host_lib, x, splits=S, kernel=WIDE, counters=True)
    torch.testing.assert_close(fused.run().float(), ref.float(), atol=1e-3, rtol=8e-3)
    assert (fused.counters == 0).all()
