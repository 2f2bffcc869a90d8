"""The C-ABI library without a GPU: it loads, exports what include/zorro_fca.h declares,
sizes workspaces and rejects bad arguments before any launch."""

import ctypes
import os
import re

import pytest

from arctic_platform_amd import _lib
from arctic_platform_amd.forest import make_plan

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build_library()
    return _lib.load_library()


def test_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "zorro_fca.h")).read()
    declared = set(re.findall(r"^(?:int|const char\*)\s+(fca_\w+)\s*\(", header, flags=re.M))
    assert declared == set(_lib.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.fca_version() == 105


def test_struct_sizes_match_header():
    assert ctypes.sizeof(_lib.FcaPlan) == 9 * 4
    assert ctypes.sizeof(_lib.FcaMetaLayout) == 18 * 8
    assert ctypes.sizeof(_lib.FcaTensors) == 112


def test_workspace_sizes(lib):
    plan = make_plan(512, 320, 32, 8, 128, chunk_tokens=512, max_levels=4)
    layout = _lib.FcaMetaLayout()
    assert lib.fca_meta_describe(ctypes.byref(plan), ctypes.byref(layout)) == 0
    assert layout.max_partials == 320 * 16 // 512 + 4 + 2  # chunks + discovered levels + declared group + leaf
    assert layout.max_items == 512 * layout.max_partials
    nm, no, nl = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    assert lib.fca_workspace_bytes(ctypes.byref(plan), ctypes.byref(nm), ctypes.byref(no), ctypes.byref(nl)) == 0
    assert nm.value == layout.total_int32 * 4
    # one row per (partial slot, query head), then 32 rows for each of up to 1024 pairs of waves
    # that attend an item together
    rows = 512 * layout.max_partials * 32 + 32 * 1024
    assert no.value == rows * 128 * 2  # half-precision rows
    assert nl.value == rows * 2 * 4  # {lse, scale}
    tiny = make_plan(2, 4, 8, 2, 64, chunk_tokens=32, max_levels=1)  # at most 2 * 5 * 2 tickets: 11 pairs of waves
    assert lib.fca_workspace_bytes(ctypes.byref(tiny), None, ctypes.byref(no), ctypes.byref(nl)) == 0
    assert no.value == (2 * 5 * 8 + 32 * 11) * 64 * 2 and nl.value == (2 * 5 * 8 + 32 * 11) * 8


@pytest.mark.parametrize(
    "kw,fragment",
    [
        (dict(chunk_tokens=100), "chunk_tokens"),
        (dict(chunk_tokens=2048), "chunk_tokens"),
        (dict(rows_per_item=48), "rows_per_item"),
        (dict(max_levels=9), "max_levels"),
        (dict(head_dim=96), "head_dim"),
        (dict(head_dim=512), "head_dim"),
        (dict(head_dim=256, rows_per_item=64), "head_dim 256"),
        (dict(num_q_heads=30), "num_q_heads"),
    ],
)
def test_bad_plans_are_rejected(lib, kw, fragment):
    base = dict(num_seqs=4, max_blocks=8, num_q_heads=32, num_kv_heads=8, head_dim=128)
    tiling = dict(chunk_tokens=512, rows_per_item=32, max_levels=4)
    for k, v in kw.items():
        (base if k in base else tiling)[k] = v
    plan = make_plan(**base, **tiling)
    rc = lib.fca_meta_describe(ctypes.byref(plan), ctypes.byref(_lib.FcaMetaLayout()))
    assert rc < 0 and fragment in lib.fca_last_error().decode()


def test_block_size_and_null_pointers(lib):
    plan = make_plan(4, 8, 32, 8, 128)
    plan.block_size = 32
    assert lib.fca_meta_describe(ctypes.byref(plan), ctypes.byref(_lib.FcaMetaLayout())) == -2
    plan.block_size = 16
    assert lib.fca_build_metadata(ctypes.byref(plan), None, 8, None, None, None) == -1
    assert "non-NULL" in lib.fca_last_error().decode()
    t = _lib.FcaTensors()
    assert lib.fca_decode_step(ctypes.byref(plan), ctypes.byref(t), None, None, None, None, 0, 0, 0, None, None) == -1


def test_row_entry_points_check_their_arguments(lib):
    plan = make_plan(4, 8, 32, 8, 128)
    one = ctypes.c_void_p(16)  # never dereferenced: the checks come first
    # a row table needs the number of table rows
    assert lib.fca_build_metadata_rows(ctypes.byref(plan), one, 8, 0, one, None, one, one, 0, None) == -1
    assert "table_rows" in lib.fca_last_error().decode()
    assert lib.fca_build_metadata_rows(ctypes.byref(plan), None, 8, 2, one, None, one, one, 0, None) == -1
    assert lib.fca_rows_from_query_runs(one, one, 0, 4, 8, one, one, one, None) == -1
    assert lib.fca_rows_from_query_runs(one, one, 1 << 20, 4, 1 << 12, one, one, one, None) == -2  # group ids need 32 bits
    assert lib.fca_rows_from_query_runs(None, None, 2, 0, 8, None, None, None, None) == 0  # nothing to do
    assert lib.fca_rows_from_query_runs(None, one, 2, 4, 8, one, one, one, None) == -1


def test_operators_refuse_cpu_tensors():
    import torch

    from arctic_platform_amd.forest import build_forest_metadata

    with pytest.raises(RuntimeError, match="GPU"):
        build_forest_metadata(
            torch.zeros(2, 4, dtype=torch.int32), torch.ones(2, dtype=torch.int32), num_q_heads=8, num_kv_heads=2, head_dim=64
        )


def test_operators_check_layouts_before_the_device():
    import torch

    from arctic_platform_amd.cache import append_kv
    from arctic_platform_amd.forest import build_forest_metadata

    table = torch.zeros(2, 4, dtype=torch.int32)
    with pytest.raises(ValueError, match="contiguous"):  # every other length: a strided view
        build_forest_metadata(table, torch.ones(4, dtype=torch.int32)[::2], num_q_heads=8, num_kv_heads=2, head_dim=64)
    kv = torch.zeros(2, 4, 2, 16 * 64 * 2, dtype=torch.bfloat16)[..., ::2]  # tiles not contiguous
    rows = torch.zeros(3, 2, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="contiguous tiles"):
        append_kv(rows, rows, kv, torch.zeros(3, dtype=torch.int64))


def test_header_is_plain_c_and_links(tmp_path):
    """include/zorro_fca.h compiles as C99 and as C++, and a C program that only sizes a
    workspace links against the library and runs without a GPU."""
    import shutil
    import subprocess

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "probe.c"
    src.write_text(
        '#include "zorro_fca.h"\n#include <stdio.h>\n'
        "int main(void) {\n"
        "  fca_plan p = {512, 320, 32, 8, 128, 16, 1024, 32, 4};\n"
        "  size_t m = 0, o = 0, l = 0;\n"
        "  if (fca_workspace_bytes(&p, &m, &o, &l) != 0) { puts(fca_last_error()); return 1; }\n"
        '  printf("%d %zu %zu %zu\\n", fca_version(), m, o, l);\n'
        "  /* the trainer's layout array is host code: two prompts of 3 and 2 tokens, responses 2, 1 | 4 */\n"
        "  int32_t prompts[2] = {3, 2}, sizes[2] = {2, 1}, responses[3] = {2, 1, 4};\n"
        "  int64_t n = 0;\n"
        "  int32_t layout[512];\n"
        "  if (fca_split_layout_ints(12, &n) != 0 || n > 512) return 2;\n"
        "  if (fca_split_layout_build(2, prompts, sizes, responses, 12, 0, 0, layout) != 0) { puts(fca_last_error()); return 3; }\n"
        '  for (int i = 0; i < 12; ++i) printf("%d ", layout[i]);\n'
        "  p.head_dim = 96;\n"
        "  return fca_workspace_bytes(&p, &m, &o, &l) == 0;  /* must be refused */\n"
        "}\n"
    )
    inc, libdir = os.path.join(root, "include"), os.path.join(root, "arctic_platform_amd")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-x", "c", os.path.join(inc, "zorro_fca.h")], check=True)
    subprocess.run([shutil.which("g++") or gcc, "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", os.path.join(inc, "zorro_fca.h")], check=True)
    exe = tmp_path / "probe"
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", f"-I{inc}", str(src), f"-L{libdir}", "-lzorro_fca", f"-Wl,-rpath,{libdir}", "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert int(out[0]) >= 1 and int(out[2]) == (512 * (320 * 16 // 1024 + 6) * 32 + 32 * 1024) * 128 * 2
    # lim of every key: a prompt token is seen up to the end of its group, a response token up to its own end
    assert [int(x) for x in out[4:16]] == [6, 6, 6, 5, 5, 6, 12, 12, 12, 12, 12, 12]


def test_attention_and_cache_entry_points_refuse_bad_tensors(lib):
    """Every check that stands between a caller's mistake and a kernel launch: the calls below
    must come back with an error code and a message, never reach a launch (there is no GPU here:
    a call that got that far would report a HIP error instead)."""
    plan = make_plan(4, 8, 32, 8, 128)
    ok = 1 << 20  # an address that is 16-byte aligned and never dereferenced

    def tensors(**kw):
        t = _lib.FcaTensors(ok, 32 * 128, 128, ok, ok + (1 << 16), 8 * 16 * 128, 16 * 128, _lib.FCA_BF16, 0, ok, 8, None, None, 0.1)
        for k, v in kw.items():
            setattr(t, k, v)
        return t

    def decode(t, meta=ok, po=ok, pl=ok, out=ok, out_dtype=_lib.FCA_BF16):
        return lib.fca_decode_step(ctypes.byref(plan), ctypes.byref(t), meta, po, pl, out, 32 * 128, 128, out_dtype, None, None)

    cases = [
        (tensors(q_dev=ok + 2), "q must be 16-byte aligned"),
        (tensors(q_head_stride=100), "strides that are multiples of 8"),
        (tensors(k_cache_dev=ok + 8), "KV cache planes must be 16-byte aligned"),
        (tensors(kv_dtype=7), "kv_dtype 7"),
        (tensors(kv_head_stride=16 * 64), "smaller than one tile"),
        (tensors(block_table_stride=4), "block_table_stride 4 is smaller than max_blocks 8"),
        (tensors(block_table_dev=None), "must be non-NULL"),
    ]
    for t, fragment in cases:
        assert decode(t) < 0
        assert fragment in lib.fca_last_error().decode(), (fragment, lib.fca_last_error())
    assert decode(tensors(), po=ok + 4) == -1 and "partial workspaces must be 16-byte aligned" in lib.fca_last_error().decode()
    assert decode(tensors(), meta=None) == -1
    # the merge: output type and pointers
    assert lib.fca_merge(ctypes.byref(plan), ok, ok, ok, ok, 32 * 128, 128, 5, None, None) == -2
    assert lib.fca_merge(ctypes.byref(plan), ok, ok, ok, None, 32 * 128, 128, _lib.FCA_BF16, None, None) == -1
    # the static entry point refuses plans whose partial rows do not fit its array
    big = make_plan(4096, 512, 32, 8, 128, chunk_tokens=32)
    assert lib.fca_decode_step_static(ctypes.byref(big), ctypes.byref(tensors(block_table_stride=512)), ok, ok, 32 * 128, 128, _lib.FCA_BF16, None, None) == -2
    assert "static scratch" in lib.fca_last_error().decode()
    # cache writer and reader
    def append(fn=lib.fca_append_kv, key=ok, tstride=8 * 128, hstride=128, tokens=3, heads=8, d=128, slots=ok, kc=ok, bstride=8 * 16 * 128, hs=16 * 128, dt=_lib.FCA_BF16):
        return fn(key, ok, tstride, hstride, tokens, heads, d, slots, kc, ok + (1 << 16), bstride, hs, dt, None, None, None)

    assert append(tokens=0) == 0  # nothing to do
    for kw, fragment in [
        (dict(tokens=-1), "num_tokens must be >= 0"),
        (dict(d=96), "head_dim 96"),
        (dict(dt=3), "kv_dtype 3"),
        (dict(key=ok + 8), "key and value must be 16-byte aligned"),
        (dict(tstride=100), "multiples of 8"),
        (dict(slots=None), "must be non-NULL"),
        (dict(hs=16 * 64), "at least one tile"),
    ]:
        for fn in (lib.fca_append_kv, lib.fca_gather_kv):
            assert append(fn=fn, **kw) < 0
            assert fragment in lib.fca_last_error().decode(), (fragment, lib.fca_last_error())
    # the measurement hook takes its events as a pair
    assert lib.fca_time_next_attention(ok, None) == -1
    assert lib.fca_time_next_attention(None, None) == 0
    assert lib.fca_calibration_copy(ok, ok + 4, 64, None) == -1


def test_split_entry_points_refuse_bad_tensors(lib):
    ok = 1 << 20
    plan = _lib.FcaSplitPlan(100, 8, 2, 128)

    def forward(q=ok, qs=8 * 128, ks=2 * 128, layout=ok, scale=0.1, ws=ok, out_stride=8 * 128, lse=ok):
        return lib.fca_split_attention_forward(ctypes.byref(plan), q, qs, ok, ks, ok, 2 * 128, layout, scale, ws, ok, out_stride, lse, None)

    for kw, fragment in [
        (dict(scale=0.0), "scale must be positive"),
        (dict(q=ok + 2), "q must be 16-byte aligned"),
        (dict(qs=7 * 128), "at least heads * head_dim"),
        (dict(ks=100), "k must be"),
        (dict(out_stride=4), "out must be"),
        (dict(layout=None), "layout, workspace and lse"),
        (dict(lse=ok + 4), "layout, workspace and lse"),
    ]:
        assert forward(**kw) < 0
        assert fragment in lib.fca_last_error().decode(), (fragment, lib.fca_last_error())
    empty = _lib.FcaSplitPlan(0, 8, 2, 128)
    assert lib.fca_split_attention_forward(ctypes.byref(empty), None, 0, None, 0, None, 0, None, 0.1, None, None, 0, None, None) == 0
    bad = _lib.FcaSplitPlan(-1, 8, 2, 128)
    assert lib.fca_split_workspace_bytes(ctypes.byref(bad), None, None) == -1
    args = [ok, 8 * 128, ok, 2 * 128, ok, 2 * 128, ok, 8 * 128, ok, 8 * 128, ok, ok, 0.1, ok, ok, 8 * 128, ok, 2 * 128, ok, 2 * 128, None]
    args[16] = 100  # dk stride (every call in this file must fail a check: with a GPU present a call that passed them all would launch on made-up addresses)
    assert lib.fca_split_attention_backward(ctypes.byref(plan), *args) == -1 and "dk must be" in lib.fca_last_error().decode()
