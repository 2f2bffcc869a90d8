"""Builds the library for the CPU emulation (emu.h): every ``csrc/*.hip`` becomes a host translation
unit, with its kernel launches and its few lines of GPU assembly replaced, and all of them are
linked into one shared library that exports the C ABI of ``include/zorro_fca.h`` with host pointers
where the real library takes device pointers.  Test infrastructure only."""

from __future__ import annotations

import hashlib
import os
import re
import shutil
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "arctic_platform_amd", "csrc")
CLANG = "/opt/rocm/lib/llvm/bin/clang++"

_LDS_HELPERS = """__device__ inline unsigned lds_address(const void* p) { return emu::lds_address(p); }
__device__ inline void load_to_lds16(const void* src, unsigned lds_slot) { emu::dma_to_lds(src, lds_slot, 16); }
__device__ inline void load_to_lds4(const void* src, unsigned lds_slot) { emu::dma_to_lds(src, lds_slot, 4); }
#define FCA_WAIT_VMCNT(n) emu::wait_vmcnt(n)
"""


def compiler() -> str | None:
    return CLANG if os.path.exists(CLANG) else shutil.which("clang++")


def transform(text: str) -> str:
    """Source of a ``.hip`` file -> source the host compiler takes."""
    # kernel<<<grid, block, 0, stream>>>(args)  ->  emu::launch(grid, block, [&] { kernel(args); })
    out, pos = [], 0
    for m in re.finditer(r"([\w:]+(?:<[^<>()]*>)?)<<<(.+?), (\w+), 0, stream>>>\(", text):
        out.append(text[pos : m.start()])
        depth, k = 1, m.end()
        while depth:
            depth += {"(": 1, ")": -1}.get(text[k], 0)
            k += 1
        out.append(f"emu::launch({m.group(2)}, {m.group(3)}, [&] {{ {m.group(1)}({text[m.end() : k - 1]}); }})")
        pos = k
    text = "".join(out) + text[pos:]
    # a zero the GPU compiler cannot see through
    text = text.replace('asm volatile("v_mov_b32 %0, 0" : "=v"(opaque_zero));', "opaque_zero = 0;")
    # direct-to-LDS loads and the wait that counts them
    start = "__device__ inline unsigned lds_address(const void* p) {"
    if start in text:
        a = text.index(start)
        b = text.index("\n", text.index("#define FCA_WAIT_VMCNT(n)")) + 1
        text = text[:a] + _LDS_HELPERS + text[b:]
    if "asm" in re.sub(r"//.*", "", text):
        raise RuntimeError("GPU assembly that the emulation build does not know how to replace")
    return text


def build(replace: dict | None = None, tag: str = "emu") -> str:
    """Returns the path of the built library.  ``replace`` maps a file name of ``csrc`` to another
    source to take in its place.  The library is named after a hash of everything that goes into
    it, is compiled in a directory of its own and moved into place when it is whole: a library
    that is there is up to date, and processes that build at the same time do not meet."""
    cxx = compiler()
    if cxx is None:
        raise RuntimeError("no clang++ to build the emulation with")
    replace = replace or {}
    flags = ["-std=c++17", "-O2", "-g", "-fPIC", "-w"]
    sources = {}
    for name in sorted(os.listdir(CSRC)):
        if name.endswith(".hip"):
            with open(replace.get(name, os.path.join(CSRC, name))) as f:
                sources[name.replace(".hip", ".cpp")] = transform(f.read())
    digest = hashlib.sha256(" ".join([cxx] + flags).encode())
    for name, text in sources.items():
        digest.update(name.encode() + b"\0" + text.encode())
    for folder in (HERE, os.path.join(HERE, "hip"), CSRC, os.path.join(ROOT, "include")):
        for name in sorted(os.listdir(folder)):
            if name.endswith((".h", ".hpp")) or name == "hooks.cpp":
                with open(os.path.join(folder, name), "rb") as f:
                    digest.update(name.encode() + b"\0" + f.read())
    out_dir = os.path.join(HERE, "_build_" + tag)
    os.makedirs(out_dir, exist_ok=True)
    so = os.path.join(out_dir, f"libzorro_fca_emu_{digest.hexdigest()[:16]}.so")
    if os.path.exists(so):
        return so
    work = tempfile.mkdtemp(prefix="work_", dir=out_dir)
    try:
        jobs = []
        for name, text in sources.items():
            cpp = os.path.join(work, name)
            with open(cpp, "w") as f:
                f.write(text)
            obj = cpp[:-4] + ".o"
            jobs.append((subprocess.Popen([cxx, *flags, "-c", f"-I{HERE}", f"-I{CSRC}", f"-I{ROOT}/include", cpp, "-o", obj]), obj))
        hooks = os.path.join(work, "hooks.o")
        jobs.append((subprocess.Popen([cxx, "-std=c++17", "-O2", "-fPIC", "-w", "-c", f"-I{HERE}", os.path.join(HERE, "hooks.cpp"), "-o", hooks]), hooks))
        if any(p.wait() for p, _ in jobs):
            raise RuntimeError("the emulation build failed to compile")
        whole = os.path.join(work, "lib.so")
        subprocess.run([cxx, "-shared", "-o", whole] + [o for _, o in jobs], check=True)
        os.replace(whole, so)
    finally:
        shutil.rmtree(work, ignore_errors=True)
    for name in os.listdir(out_dir):  # libraries of earlier states of the sources
        if name.startswith("libzorro_fca_emu") and os.path.join(out_dir, name) != so:
            os.unlink(os.path.join(out_dir, name))
    return so
