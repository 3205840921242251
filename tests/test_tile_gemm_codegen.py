"""What the tile GEMM's relaxed step barrier relies on, checked in the generated code.

A producer wave of ``tile_gemm_kernel`` with the codebook in LDS ends a step with
``s_waitcnt lgkmcnt(N); s_barrier`` where N is the number of codebook lookups it issued after its two
stores into the W tile (``block_sync_lds_keep`` in ``csrc/gemm_tile.hpp``).  LDS operations of a wave
complete in order, so the stores are done when at most N operations are outstanding -- provided the
compiler kept the stores in front of the lookups, issued no other LDS operation behind them, and has
no scalar or flat load in flight whose return would be counted out of order.  The source pins that
order with a compiler barrier; this test compiles the VQ tile GEMM for gfx950 (device code only, no
GPU needed, about a minute) and reads the order off the assembly of every instantiation.
"""

import re
import shutil
import subprocess

import pytest

from neuropress_amd import build


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    """The gfx950 assembly of the VQ tile GEMM, compiled once for the tests of this file."""
    if shutil.which("hipcc") is None and not build.Path("/opt/rocm/bin/hipcc").exists():
        pytest.skip("needs hipcc")
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    out = tmp_path_factory.mktemp("codegen") / "vq_gemm.s"
    cmd = [hipcc, *build.CXXFLAGS, *build.DEVICE_FLAGS, "-S", "--cuda-device-only",
           str(build.CSRC / "vq_gemm.hip"), "-o", str(out)]  # fmt: skip
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    return out.read_text().split("\n")


def test_relaxed_step_barriers_follow_stores_then_lookups(assembly):
    lines = assembly
    starts = [i for i, ln in enumerate(lines) if re.match(r"^_ZN5npamd16tile_gemm_kernel\S*: ;", ln)]
    assert len(starts) >= 100  # every (activation, width, vector length, tokens band, LDS) instantiation
    kernels_with_relaxed, relaxed = 0, 0
    for i in starts:
        name = lines[i].split(":")[0]
        end = next(j for j in range(i, len(lines)) if lines[j].startswith(".Lfunc_end"))
        body = lines[i:end]
        found = 0
        for k, ln in enumerate(body[:-1]):
            m = re.search(r"s_waitcnt lgkmcnt\((\d+)\)", ln)
            if not (m and int(m.group(1)) > 0 and "s_barrier" in body[k + 1]):
                continue
            keep = int(m.group(1))
            ops = []
            j = k - 1
            while j >= 0 and "s_barrier" not in body[j]:
                op = re.match(r"\s+(ds_\w+|s_load\w+|s_buffer_load\w+|flat_\w+)", body[j])
                if op:
                    ops.append(op.group(1))
                j -= 1
            ops.reverse()
            assert not [o for o in ops if not o.startswith("ds_")], (name, ops)  # nothing counted out of order
            assert len(ops) > keep and all(o.startswith("ds_read") for o in ops[-keep:]), (name, ops)
            assert all(o.startswith("ds_write") for o in ops[:-keep]), (name, ops)  # the stores, and only them, in front
            found += 1
        if found:
            # the LDS-codebook variant (last template argument true), eight unrolled steps
            assert name.endswith("ELb1EEEvNS_9GemmShapeENT0_4ArgsE") and found == 8, (name, found)
            kernels_with_relaxed += 1
            relaxed += found
    assert kernels_with_relaxed >= 40 and relaxed == 8 * kernels_with_relaxed


def test_nothing_but_the_lds_direct_loads_touches_m0(assembly):
    """The x tile is fetched with ``s_mov_b32 m0, <LDS address>; global_load_lds_dwordx4`` in an asm
    statement that cannot declare m0 as clobbered (the compiler reserves it).  That is sound only
    while the compiler itself keeps nothing in m0 inside ``tile_gemm_kernel``: every instruction of
    the generated kernels that names m0 must sit inside one of those asm statements."""
    lines = assembly
    starts = [i for i, ln in enumerate(lines) if re.match(r"^_ZN5npamd16tile_gemm_kernel\S*: ;", ln)]
    assert starts
    checked = 0
    for i in starts:
        end = next(j for j in range(i, len(lines)) if lines[j].startswith(".Lfunc_end"))
        in_asm = False
        for ln in lines[i:end]:
            if "#ASMSTART" in ln:
                in_asm = True
            elif "#ASMEND" in ln:
                in_asm = False
            elif re.search(r"\bm0\b", ln.split(";")[0]):
                assert in_asm, ln
                checked += 1
    assert checked > 0


@pytest.fixture(scope="module")
def assembly_wide(tmp_path_factory):
    """The gfx950 assembly of the 128-column tile GEMM (csrc/gemm_tile2.hip)."""
    if shutil.which("hipcc") is None and not build.Path("/opt/rocm/bin/hipcc").exists():
        pytest.skip("needs hipcc")
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    out = tmp_path_factory.mktemp("codegen") / "gemm_tile2.s"
    cmd = [hipcc, *build.CXXFLAGS, *build.DEVICE_FLAGS, "-S", "--cuda-device-only",
           str(build.CSRC / "gemm_tile2.hip"), "-o", str(out)]  # fmt: skip
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    return out.read_text().split("\n")


def test_the_wide_kernel_loads_everything_into_lds_and_leaves_m0_to_its_transfers(assembly_wide):
    """``tile2_gemm_kernel`` brings x tiles, indices, codebook rows and packed bytes into LDS with
    ``s_mov_b32 m0, <LDS address>; global_load_lds_dword[x4]`` asm statements and counts them by hand
    (``s_waitcnt vmcnt(n)``).  Sound only while (a) the compiler keeps nothing of its own in m0 and (b)
    every vector-memory load of the main loop is one of those transfers, so that the hand-written counts
    see all of a wave's loads: outside asm statements the kernels may load from global memory only where
    the compiler's own waits cover it (bias, the other half's tile, and the look at the tile word in front of
    the last step, which only makes the hand-written waits behind it stricter)."""
    lines = assembly_wide
    starts = [i for i, ln in enumerate(lines) if re.match(r"^_ZN5npamd17tile2_gemm_kernel\S*: ;", ln)]
    assert len(starts) >= 20  # VQ and int4 / int8 producers x activation dtypes x row tiles
    for i in starts:
        name = lines[i].split(":")[0]
        end = next(j for j in range(i, len(lines)) if lines[j].startswith(".Lfunc_end"))
        in_asm, transfers, spills = False, 0, 0
        for ln in lines[i:end]:
            code = ln.split(";")[0]
            if "#ASMSTART" in ln:
                in_asm = True
            elif "#ASMEND" in ln:
                in_asm = False
            elif re.search(r"\bm0\b", code):
                assert in_asm, (name, ln)
            if in_asm and "global_load_lds_dword" in code:
                transfers += 1
            if re.match(r"\s+scratch_(load|store)", code):
                spills += 1
        assert transfers >= 10, (name, transfers)
        assert spills == 0, (name, spills)  # 256 registers per lane hold the wave tile: nothing goes to scratch


@pytest.fixture(scope="module")
def assembly_gemv(tmp_path_factory):
    """The gfx950 assembly of the fused decode GEMV (csrc/vq_gemv.hip)."""
    if shutil.which("hipcc") is None and not build.Path("/opt/rocm/bin/hipcc").exists():
        pytest.skip("needs hipcc")
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    out = tmp_path_factory.mktemp("codegen") / "vq_gemv.s"
    cmd = [hipcc, *build.CXXFLAGS, *build.DEVICE_FLAGS, "-S", "--cuda-device-only",
           str(build.CSRC / "vq_gemv.hip"), "-o", str(out)]  # fmt: skip
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    return out.read_text().split("\n")


def test_the_gemv_leaves_m0_to_its_codebook_copy(assembly_gemv):
    """``fused_gemv_kernel`` copies a codebook into LDS with ``s_mov_b32 m0, ...;
    global_load_lds_dwordx4`` statements and waits for them with ``s_waitcnt vmcnt(0)`` inside the same
    asm block sequence; nothing else in the kernels may name m0."""
    lines = assembly_gemv
    starts = [i for i, ln in enumerate(lines) if re.match(r"^_ZN5npamd17fused_gemv_kernel\S*: ;", ln)]
    assert len(starts) >= 50
    with_copy = 0
    for i in starts:
        name = lines[i].split(":")[0]
        end = next(j for j in range(i, len(lines)) if lines[j].startswith(".Lfunc_end"))
        in_asm, transfers = False, 0
        for ln in lines[i:end]:
            code = ln.split(";")[0]
            if "#ASMSTART" in ln:
                in_asm = True
            elif "#ASMEND" in ln:
                in_asm = False
            elif re.search(r"\bm0\b", code):
                assert in_asm, (name, ln)
            if in_asm and "global_load_lds_dwordx4" in code:
                transfers += 1
        with_copy += transfers > 0
    assert with_copy >= 20  # the variants that keep a table in LDS
