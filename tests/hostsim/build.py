"""Builds ``_build/libflexhip_hostsim.so``: the package's non-MFMA kernels and their C entry points compiled
for the CPU against the stand-in ``hip/hip_runtime.h`` of this directory (test infrastructure, see there).

The sources are the package's own ``csrc/*.hip`` files with two textual changes, both forced by syntax that
only a HIP compiler accepts: a kernel launch ``k<<<grid, block, lds, stream>>>(args)`` becomes
``hostsim::launch(grid, block, lds, [=] { k(args); })`` and ``extern __shared__ T name[];`` becomes a
pointer to the simulation's dynamic LDS.  Everything else (kernels, device helpers, host-side launch code,
argument checks) is compiled as it stands."""
from __future__ import annotations

import os
import re
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "flextrain_amd", "csrc")
OUT = os.path.join(HERE, "_build")
LIB = os.path.join(OUT, "libflexhip_hostsim.so")
CLANG = "/opt/rocm/lib/llvm/bin/clang++"
SOURCES = ("rmsnorm.hip", "rope.hip", "glu.hip", "softmax_ce.hip", "adamw.hip", "moe_route.hip", "moe_data.hip", "embed.hip")


def _match_forward(text, i, open_ch, close_ch):
    """Index just past the bracket that closes the one at ``text[i]``."""
    depth = 0
    while True:
        c = text[i]
        if c == open_ch:
            depth += 1
        elif c == close_ch:
            depth -= 1
            if depth == 0:
                return i + 1
        i += 1


def _split_top(args):
    parts, depth, cur = [], 0, ""
    for c in args:
        if c in "([{<":
            depth += 1
        elif c in ")]}>":
            depth -= 1
        if c == "," and depth == 0:
            parts.append(cur.strip())
            cur = ""
        else:
            cur += c
    parts.append(cur.strip())
    return parts


def rewrite_launches(text):
    out, pos = "", 0
    while True:
        i = text.find("<<<", pos)
        if i < 0:
            return out + text[pos:]
        # the kernel expression to the left: identifier, optionally with a template argument list
        j = i
        if text[j - 1] == ">":
            depth, j = 0, j - 1
            while True:
                if text[j] == ">":
                    depth += 1
                elif text[j] == "<":
                    depth -= 1
                    if depth == 0:
                        break
                j -= 1
        while j > 0 and (text[j - 1].isalnum() or text[j - 1] in "_:"):
            j -= 1
        kernel = text[j:i]
        k = text.index(">>>", i)
        config = _split_top(text[i + 3:k]) + ["0", "nullptr"]
        a = k + 3
        while text[a].isspace() or text[a] == "\\":
            a += 1
        assert text[a] == "(", f"launch of {kernel} without an argument list"
        b = _match_forward(text, a, "(", ")")
        out += text[pos:j] + f"hostsim::launch(dim3({config[0]}), dim3({config[1]}), (size_t)({config[2]}), [=]() {{ {kernel}{text[a:b]}; }})"
        pos = b


def rewrite_dynamic_lds(text):
    return re.sub(r"extern\s+__shared__\s+(?:__align__\(\d+\)\s+)?([A-Za-z_0-9:]+)\s+(\w+)\[\];",
                  r"\1* \2 = reinterpret_cast<\1*>(hostsim::g_dynamic_lds);", text)


def build(force=False):
    os.makedirs(OUT, exist_ok=True)
    inputs = [os.path.join(CSRC, f) for f in SOURCES] + [os.path.join(CSRC, "common.h"), os.path.join(HERE, "hostsim.cpp"),
                                                            os.path.join(HERE, "hip", "hip_runtime.h"), os.path.abspath(__file__)]
    if not force and os.path.exists(LIB) and all(os.path.getmtime(LIB) >= os.path.getmtime(p) for p in inputs):
        return LIB
    objects = []
    for name in SOURCES:
        text = open(os.path.join(CSRC, name)).read()
        cpp = os.path.join(OUT, name.replace(".hip", "_hostsim.cpp"))
        with open(cpp, "w") as f:
            f.write(rewrite_dynamic_lds(rewrite_launches(text)))
        objects.append(cpp)
    cmd = [CLANG, "-std=c++17", "-O1", "-g", "-fPIC", "-shared", "-D__HIP__", "-Wno-everything", "-I", HERE, "-I", CSRC,
           "-I", os.path.join(ROOT, "include"), "-o", LIB, os.path.join(HERE, "hostsim.cpp")] + objects
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("host simulation build failed:\n" + proc.stderr[-6000:])
    return LIB


if __name__ == "__main__":
    print(build(force=True))
