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
SOURCES = ("rmsnorm.hip", "rope.hip", "glu.hip", "softmax_ce.hip", "adamw.hip", "moe_route.hip", "moe_data.hip", "embed.hip",
           "gemm.hip", "gemm_glu.hip", "gemm_ksum.hip", "gemm_segments.hip", "grouped_gemm.hip", "stream.hip")
HEADERS = ("common.h", "gemm_core.h", "gemm_core2.h")


def _marker():
    import pytest

    return pytest.mark.skipif(not os.path.exists(CLANG), reason=f"the host simulation is compiled with {CLANG}")


needs_host_clang = _marker()


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
    return re.sub(r"extern\s+__shared__\s+(?:__align__\(\d+\)\s+)?([A-Za-z_0-9: ]+?)\s+(\w+)\[\];",
                  r"\1* \2 = reinterpret_cast<\1*>(hostsim::g_dynamic_lds);", text)


def rewrite_asm(text):
    """The three kinds of inline assembly in the GEMM code: the two LDS-DMA loads become calls of the
    stand-in, which queues the copy; the wait-count instructions become the call that lets the lane's
    queued copies land down to the count they name."""
    def one(m):
        body = m.group(1)
        if "global_load_lds_dwordx4 %1, off" in body:
            return "hostsim::lds_dma16(lds_addr, gptr);"
        if "global_load_lds_dwordx4 %1, %2" in body:
            return "hostsim::lds_dma16(lds_addr, reinterpret_cast<const char*>(sbase) + lane_off);"
        assert "s_waitcnt" in body, f"inline assembly the host simulation has no stand-in for: {body[:80]}"
        count = re.search(r"vmcnt\((\d+|%0)\)", body)
        if count is None:
            return "((void)0);"
        n = count.group(1)
        if n == "%0":
            n = re.search(r'"n"\((.*?)\)\s*:', body).group(1)
        return f"hostsim::wait_vmcnt({n});"
    return re.sub(r"asm volatile\((.*?)\);", one, text)


# Entry points whose launches take part in multi-stream schedules declare the bytes they read and write to
# the happens-before check (order.cpp) before anything else: (pointer, bytes, is_write) triples.
DECLARED_ACCESSES = {
    "fx_adamw_step": [("g", "n * elem_size(g_dt)", 0), ("p", "n * elem_size(p_dt)", 1), ("m", "n * elem_size(state_dt)", 1),
                      ("v", "n * elem_size(state_dt)", 1), ("p_bf16_out", "n * 2", 1)],
}


def rewrite_declared_accesses(text):
    for name, accesses in DECLARED_ACCESSES.items():
        m = re.search(r'extern "C" int ' + name + r"\(", text)
        if m is None:
            continue
        brace = text.index("{", _match_forward(text, m.end() - 1, "(", ")"))
        lo = ", ".join(f"(uint64_t)(uintptr_t)({ptr})" for ptr, _, _ in accesses)
        nbytes = ", ".join(f"(uint64_t)(n > 0 ? ({size}) : 0)" for _, size, _ in accesses)
        writes = ", ".join(str(w) for _, _, w in accesses)
        snippet = (f"\n    {{ const uint64_t lo__[] = {{{lo}}}, bytes__[] = {{{nbytes}}}; const int write__[] = {{{writes}}};"
                   f"\n      if (hostsim_order_enqueue((uint64_t)(uintptr_t)stream, \"{name}\", {len(accesses)}, lo__, bytes__, write__))"
                   f" FX_FAIL(\"{name}: stream order violation (host simulation)\"); }}")
        text = text[:brace + 1] + snippet + text[brace + 1:]
    return text


def rewrite_lockstep(text):
    """A GPU wave runs its lanes in lockstep, so a wave may stage values in LDS and read its neighbours'
    values back with no barrier in between; fibers do not.  The sources mark those points with comment lines
    that start with ``// lockstep:``; here each becomes a wave-level rendezvous."""
    return re.sub(r"^(\s*)// lockstep:", r"\1hostsim::sync_wave();  // lockstep:", text, flags=re.M)


def build(force=False):
    os.makedirs(OUT, exist_ok=True)
    inputs = [os.path.join(CSRC, f) for f in SOURCES + HEADERS] + [os.path.join(HERE, "hostsim.cpp"), os.path.join(HERE, "order.cpp"),
                                                                      os.path.join(HERE, "hip", "hip_runtime.h"), os.path.abspath(__file__)]
    if not force and os.path.exists(LIB) and all(os.path.getmtime(LIB) >= os.path.getmtime(p) for p in inputs):
        return LIB
    objects = []
    for name in HEADERS:                 # the headers with inline assembly are rewritten too and found first
        with open(os.path.join(OUT, name), "w") as f:
            f.write(rewrite_lockstep(rewrite_asm(open(os.path.join(CSRC, name)).read())))
    for name in SOURCES:
        text = open(os.path.join(CSRC, name)).read()
        cpp = os.path.join(OUT, name.replace(".hip", "_hostsim.cpp"))
        with open(cpp, "w") as f:
            f.write(rewrite_declared_accesses(rewrite_lockstep(rewrite_asm(rewrite_dynamic_lds(rewrite_launches(text))))))
        objects.append(cpp)
    flags = [CLANG, "-std=c++17", "-O2", "-g", "-fPIC", "-D__HIP__", "-Wno-everything", "-I", HERE, "-I", OUT, "-I", CSRC,
             "-I", os.path.join(ROOT, "include")]
    units = [os.path.join(HERE, "hostsim.cpp"), os.path.join(HERE, "order.cpp")] + objects

    def compile_one(src):
        obj = os.path.join(OUT, os.path.basename(src) + ".o")
        proc = subprocess.run(flags + ["-c", src, "-o", obj], capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"host simulation build failed ({os.path.basename(src)}):\n" + proc.stderr[-6000:])
        return obj

    from concurrent.futures import ThreadPoolExecutor

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:      # one compiler process per source
        objs = list(pool.map(compile_one, units))
    # linked under a temporary name and renamed: a process that has the old library mapped keeps it
    proc = subprocess.run([CLANG, "-shared", "-o", LIB + ".tmp"] + objs, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("host simulation link failed:\n" + proc.stderr[-6000:])
    os.replace(LIB + ".tmp", LIB)
    return LIB


if __name__ == "__main__":
    print(build(force=True))
