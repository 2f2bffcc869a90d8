"""Properties of the compiled attention kernels that the measured speed rests on, checked
on the generated gfx950 assembly (no GPU needed): the kernels use no scratch memory, and
inside the tile loop of the 32-row kernel no wait covers the tile that was requested last.

gfx9 counts outstanding vector memory operations in order and the compiler sizes every
wait for the shortest path to it, so a load that is issued on some paths only, or a value
that has to be parked behind a load, silently turns a counted wait into a wait for
everything in flight.  Nothing fails when that happens; the kernel just streams slower.
"""

import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "arctic_platform_amd", "csrc")
FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only"]


@pytest.fixture(scope="module")
def hipcc():
    exe = shutil.which("hipcc") or ("/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else None)
    if exe is None:
        pytest.skip("no hipcc")
    return exe


def _functions(asm):
    """name -> body of every kernel in an assembly listing."""
    out = {}
    for m in re.finditer(r"^(_ZN3fca\w+):[^\n]*\n(.*?)^\.Lfunc_end", asm, flags=re.M | re.S):
        out[m.group(1)] = m.group(2)
    return out


def test_attention_kernels_use_no_scratch(hipcc, tmp_path):
    # (the fp32 kernel keeps 32 rows of running maxima, sums and accumulators in registers,
    # and the merge its partial rows: in scratch they would be memory traffic per token)
    sources = (("fca_attend32.hip", 10), ("fca_attend.hip", 12), ("fca_attend_f32.hip", 2), ("fca_merge.hip", 11))
    jobs = [
        subprocess.Popen(
            [hipcc, *FLAGS, "-c", "-Rpass-analysis=kernel-resource-usage", os.path.join(CSRC, src), "-o", str(tmp_path / (src + ".o"))],
            stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, cwd=CSRC,
        )
        for src, _ in sources
    ]
    for (src, count), job in zip(sources, jobs):
        _, stderr = job.communicate()
        assert job.returncode == 0, stderr[-2000:]
        names = re.findall(r"Function Name: (\S+)", stderr)
        sizes = [int(n) for n in re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", stderr)]
        assert len(names) == len(sizes) == count, (src, names)
        for name, size in zip(names, sizes):
            if "ILi256E" in name:
                # head size 256 (one row tile, one tile buffer): the bf16 instance parks a few
                # pointers in scratch; anything beyond that would be tile data
                assert size <= 128, (name, size)
            else:
                assert size == 0, (name, size)


def test_tile_loop_of_the_32_row_kernel_keeps_a_tile_in_flight(hipcc, tmp_path):
    out = tmp_path / "a32.s"
    res = subprocess.run([hipcc, *FLAGS, "-S", os.path.join(CSRC, "fca_attend32.hip"), "-o", str(out)], capture_output=True, text=True, cwd=CSRC)
    assert res.returncode == 0, res.stderr[-2000:]
    kernels = _functions(out.read_text())
    # <head size 128, bf16, streaming, two tile buffers>: the kernel of the headline configuration
    # (8 K + 2 x 4 V loads of 16 bytes per lane and tile; every wait inside the loop leaves at least
    # the loads of one whole tile outstanding); the fp8 instances: tiles of 8 loads, one of them
    # outstanding at every wait with two tile buffers, two of them with three
    for template_args, loads_per_tile, tiles_left in (("ILi128ELb0ELb1ELi2E", 16, 1), ("ILi128ELb1ELb1ELi2E", 8, 1), ("ILi128ELb1ELb1ELi3E", 8, 2)):
        name = f"_ZN3fca19fca_attend32_kernel{template_args}EEvNS_12AttendParamsE"
        assert name in kernels, sorted(kernels)
        seen = 0
        for block in re.split(r"^\.LBB", kernels[name], flags=re.M):
            header = block.split("\n", 1)[0]
            if "Depth=2" not in header:  # the tile loop is the only loop nested inside the item loop that holds MFMAs
                continue
            if "v_mfma" not in block:
                continue
            waits = [int(n) for n in re.findall(r"s_waitcnt vmcnt\((\d+)\)", block)]
            assert waits, header
            assert min(waits) >= tiles_left * loads_per_tile, (name, header, waits)
            assert len(re.findall(r"global_load_dwordx4", block)) == loads_per_tile, (name, header)
            seen += 1
        assert seen >= 1, name


def test_merge_issues_the_loads_of_a_batch_before_it_waits(hipcc, tmp_path):
    """The merge is a chain of memory round trips with little to hide them behind, so it takes its
    partials in batches: the {lse, scale} pairs and rows of a whole batch are requested back to
    back, with no branch and no wait on the vector-memory counter between them, and so are the
    second partials of a batch.  (A loop that loads and accumulates one partial at a time
    compiles to a wait after every load.)  And it stays below 128 registers: four waves per
    SIMD, so the 4096 waves of a 512-sequence batch at 32 query heads are resident at once."""
    out = tmp_path / "merge.s"
    res = subprocess.run([hipcc, *FLAGS, "-S", os.path.join(CSRC, "fca_merge.hip"), "-o", str(out)], capture_output=True, text=True, cwd=CSRC)
    assert res.returncode == 0, res.stderr[-2000:]
    asm = out.read_text()
    kernels = {k: v for k, v in _functions(asm).items() if "fca_merge_kernel" in k}
    assert len(kernels) == 10, sorted(kernels)
    for name, body in kernels.items():
        split, f32 = re.search(r"ILi\d+ELi(\d)ELb([01])E", name).groups()
        batch = 4 if f32 == "1" or split != "1" else 6
        per_partial = 3 if f32 == "1" else 2  # 8 bytes of {lse, scale}; the lane's 16 bytes of a half-precision row, 32 of an fp32 one
        lines = [l.split(";")[0].strip() for l in body.splitlines()]
        streamed = [i for i, l in enumerate(lines) if l.startswith("global_load") and l.endswith(" nt")]
        second = [i for i, l in enumerate(lines) if l.startswith("global_load_dwordx") and not l.endswith(" nt")]
        assert len(streamed) == len(second) == batch * per_partial, (name, len(streamed), len(second))
        for group in (streamed, second):
            between = lines[group[0] : group[-1]]
            assert not [l for l in between if (l.startswith("s_waitcnt") and "vmcnt" in l) or l.startswith("s_cbranch")], name
        vgprs = int(re.search(r"\.amdhsa_kernel " + re.escape(name) + r"\n.*?\.amdhsa_next_free_vgpr (\d+)", asm, flags=re.S).group(1))
        assert vgprs <= 128, (name, vgprs)


def test_split_attention_kernels_use_no_scratch_and_keep_their_ring_in_flight(hipcc, tmp_path):
    """The dK and dV kernels of the trainer's split attention stream their operands through
    a ring of LDS stages filled by direct-to-LDS loads that stay in flight across steps.  The
    only waits on the vector-memory counter the kernels may hold are the ones written in the
    source: one for everything before the loop, the counted pair at the top of a step (wave 0
    requests one load more per step than the others), one for everything after the loop.  A
    wait the compiler adds inside the loop would drain the ring every step."""
    out = tmp_path / "split.s"
    res = subprocess.run(
        [hipcc, *FLAGS, "-S", "-Rpass-analysis=kernel-resource-usage", os.path.join(CSRC, "fca_split.hip"), "-o", str(out)],
        capture_output=True, text=True, cwd=CSRC,
    )
    assert res.returncode == 0, res.stderr[-2000:]
    sizes = re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", res.stderr)
    assert len(sizes) >= 35 and set(sizes) == {"0"}, sizes
    kernels = {k: v for k, v in _functions(out.read_text()).items() if "split_key_kernel" in k}
    assert len(kernels) == 12, sorted(kernels)  # head sizes 64 / 128 / 256 x dV / dK x without / with a sliding window
    for name, body in kernels.items():
        head_dim, dk, window = re.search(r"ILi(\d+)ELb([01])ELb([01])E", name).groups()
        slots = (3 if dk == "1" else 2) * int(head_dim) // 16
        per_wave = slots // 4
        waits = [int(n) for n in re.findall(r"s_waitcnt[^\n]*vmcnt\((\d+)\)", body)]
        assert waits == [0, per_wave, per_wave + 1, 0], (name, waits)
        assert body.count("global_load_lds_dwordx4") == 3 * per_wave, name  # two stages ahead of the loop, one inside
        # the rows' log-sum-exp and delta (wave 0) and, with a window, their positions (wave 1)
        assert body.count("global_load_lds_dword ") + body.count("global_load_lds_dword\t") == (6 if window == "1" else 3), name
