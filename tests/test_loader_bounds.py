"""Bounds audit of the GEMM tile loaders, on the CPU.

The address generation of the MFMA kernels (which byte of which operand a lane requests, in which
K-step) is plain integer C++ inside ``csrc/gemm_core2.h``.  This test lifts that code TEXTUALLY out of
the headers (the operand view and the loader structs, unchanged), puts it into a host translation unit
in which the two load instructions are recorders instead of ``global_load_lds`` / ``global_load``,
compiles it with g++ and drives every wave and lane of a workgroup through whole K loops over a sweep
of ragged shapes: every 16-byte request must lie inside its operand, every LDS write inside its stage,
and the row maps of the gathering loaders are placed against inaccessible guard pages, so a map read
one entry past either end kills the audit.  What it proves is confined to addresses (not values), which
is exactly what a GPU memory fault is made of and what no GPU parity test can see: an over-read that
lands in mapped memory changes no result."""
from __future__ import annotations

import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "flextrain_amd", "csrc")


def _block(text, head_regex):
    """The source text from the match of ``head_regex`` to the brace that closes the block it opens."""
    m = re.search(head_regex, text, flags=re.M)
    assert m, f"not found in the header: {head_regex}"
    i = text.index("{", m.end() - 1)
    depth, j = 0, i
    while True:
        depth += {"{": 1, "}": -1}.get(text[j], 0)
        j += 1
        if depth == 0:
            break
    if text[j:j + 1] == ";":
        j += 1
    return text[m.start():j]


def _line(text, needle):
    for line in text.splitlines():
        if needle in line:
            return line
    raise AssertionError(f"not found in the header: {needle}")


HARNESS = r"""
#include <sys/mman.h>
#include <unistd.h>
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <type_traits>
#define FX_DEV inline
#define __device__
#define __forceinline__ inline
using std::max;
using std::min;

namespace fx {
typedef uint16_t bf16;
struct u32x4_t { unsigned v[4]; };
constexpr int GEMM_BK = 64;

// ------------------------------------------------------------------ the recorders
static const char* g_lo[2];
static const char* g_hi[2];
static long g_requests = 0, g_bad = 0;
static unsigned g_lds_lo = 0, g_lds_hi = 0;
static char g_case[256];
static volatile unsigned g_sink = 0;

static void audit(const void* p, int bytes) {
    const char* a = reinterpret_cast<const char*>(p);
    ++g_requests;
    for (int r = 0; r < 2; ++r)
        if (g_lo[r] && a >= g_lo[r] && a + bytes <= g_hi[r]) return;
    if (g_bad++ < 5)
        fprintf(stderr, "OUT OF BOUNDS: %s: request at operand byte %lld (+%d), operand holds %lld bytes\n", g_case,
                (long long)(a - g_lo[0]), bytes, (long long)(g_hi[0] - g_lo[0]));
}
static void audit_lds(unsigned addr) {
    if (addr < g_lds_lo || addr + 1024 > g_lds_hi) {
        if (g_bad++ < 5) fprintf(stderr, "LDS OUT OF STAGE: %s: wave instruction at %u, stage [%u, %u)\n", g_case, addr, g_lds_lo, g_lds_hi);
    }
}
inline u32x4_t ldg16(const void* p) { audit(p, 16); return u32x4_t{{0u, 0u, 0u, 0u}}; }
inline void load_to_lds16_s(unsigned lane_off, const void* sbase, unsigned lds_addr) {
    audit(reinterpret_cast<const char*>(sbase) + lane_off, 16);
    audit_lds(lds_addr);
}
inline void load_to_lds16(const void* gptr, void* lds_base) {
    audit(gptr, 16);
    audit_lds((unsigned)(uintptr_t)lds_base);
}

// ------------------------------------------------------------------ lifted from the headers, unchanged
@@LIFTED@@
}  // namespace fx

using namespace fx;

// A row map whose first and last entries touch inaccessible pages.
struct GuardedMap {
    char* region = nullptr;
    size_t bytes = 0;
    int32_t* data = nullptr;
    GuardedMap(int n) {
        const size_t page = (size_t)sysconf(_SC_PAGESIZE);
        const size_t body = ((size_t)n * 4 + page - 1) / page * page;
        bytes = body + 2 * page;
        region = (char*)mmap(nullptr, bytes, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
        if (region == MAP_FAILED) { perror("mmap"); exit(2); }
        mprotect(region, page, PROT_NONE);
        mprotect(region + page + body, page, PROT_NONE);
        data = (int32_t*)(region + page + body) - n;        // the last entry ends at the guard page
    }
    ~GuardedMap() { munmap(region, bytes); }
};

static std::mt19937 rng(12345);
static int rnd(int lo, int hi) { return lo + (int)(rng() % (unsigned)(hi - lo + 1)); }

static const bf16* const FAKE = reinterpret_cast<const bf16*>(0x100000000000ull);   // never dereferenced
static const bf16* const FAKE2 = reinterpret_cast<const bf16*>(0x200000000000ull);

static void allow(int r, const bf16* base, int64_t elems) {
    g_lo[r] = reinterpret_cast<const char*>(base);
    g_hi[r] = g_lo[r] + elems * 2;
}

template <typename L, int NI, int J = 0>
static void issue_all(L& l, bf16* lds, int wave) {
    if constexpr (J < NI) {
        l.template issue<J>(lds, wave);
        issue_all<L, NI, J + 1>(l, lds, wave);
    }
}

// The K loop's use of a 64-wide loader: init once, then every full K-step in order (two stages alternate).
template <typename L, bool KG>
static void drive64(const OperandView<bf16>& op, int K, int NW, int rows_in_stage) {
    const int nfull = K / GEMM_BK;
    if (nfull == 0) return;
    for (int wave = 0; wave < NW; ++wave)
        for (int lane = 0; lane < 64; ++lane) {
            L l;
            l.init(op, wave, lane);
            for (int kt = 0; kt < nfull; ++kt) {
                bf16* stage = reinterpret_cast<bf16*>((uintptr_t)((kt & 1) ? 96 * 1024 : 0));
                g_lds_lo = (kt & 1) ? 96 * 1024 : 0;
                g_lds_hi = g_lds_lo + rows_in_stage * GEMM_BK * 2;
                if constexpr (KG) l.prepare();
                issue_all<L, L::NI>(l, stage, wave);
                if constexpr (KG) l.fetch();
            }
        }
}

template <typename L>
static void drive32(const OperandView<bf16>& op, int K, int NW, int rows_in_stage) {
    const int n = K / 32;
    for (int wave = 0; wave < NW; ++wave)
        for (int lane = 0; lane < 64; ++lane) {
            L l;
            l.init(op, wave, lane);
            for (int kt = 0; kt < n; ++kt) {
                g_lds_lo = (kt % 3) * 24 * 1024;
                g_lds_hi = g_lds_lo + rows_in_stage * 32 * 2;
                issue_all<L, L::NI>(l, reinterpret_cast<bf16*>((uintptr_t)g_lds_lo), wave);
            }
        }
}

template <int ROWS, int NT, bool MN>
static void drive_tail(const OperandView<bf16>& op, int K) {
    const int k0 = K / GEMM_BK * GEMM_BK;
    if (k0 == K) return;
    for (int tid = 0; tid < NT; ++tid) {
        Staged2<ROWS, NT> st;
        stage2_load<bf16, ROWS, NT, MN>(st, op, k0, K, tid);
    }
}

// ---- K-contiguous operand (rows x K, row stride ld): tile rows origin .. origin + ROWS, rows >= ext clamped
template <int ROWS, int NW>
static void case_kcontig(bool gathered, bool dual) {
    const int ext = rnd(1, 700), K = rnd(1, 80) * 8, ld = K + rnd(0, 4) * 8;
    const int origin = rnd(0, (ext - 1) / ROWS) * ROWS;
    const int src_rows = gathered ? rnd(1, 900) : ext;
    snprintf(g_case, sizeof g_case, "K-contiguous %dx%d waves %d ext %d origin %d K %d ld %d gathered %d dual %d", ROWS, 64, NW, ext,
             origin, K, ld, (int)gathered, (int)dual);
    GuardedMap map(ext);
    for (int i = 0; i < ext; ++i) map.data[i] = rnd(0, 9) == 0 ? rnd(-5, src_rows + 5) : rnd(0, src_rows - 1);   // some entries out of range
    OperandView<bf16> op{FAKE, ld, ext, origin};
    allow(0, FAKE, (int64_t)(src_rows - 1) * ld + K);
    allow(1, nullptr, 0);
    if (gathered) { op.row_map = map.data; op.map_rows = src_rows; }
    if (dual) {
        op.half = 64; op.base2 = FAKE2; op.origin = origin / 2;     // a two-matrix tile covers ROWS / 2 indices of each matrix
        allow(1, FAKE2, (int64_t)(ext - 1) * ld + K);
    }
    if (dual) drive64<TileLoader<bf16, ROWS, NW, false, true>, false>(op, K, NW, ROWS);
    else drive64<TileLoader<bf16, ROWS, NW, false, false>, false>(op, K, NW, ROWS);
    if (!dual) drive_tail<ROWS, NW * 64, false>(op, K);      // gathered or not: the K tail goes through registers
    if (NW == 4 && K % 32 == 0) {
        if (dual) drive32<Tile32Loader<bf16, ROWS, NW, false, true>>(op, K, NW, ROWS);
        else drive32<Tile32Loader<bf16, ROWS, NW, false, false>>(op, K, NW, ROWS);
    }
}

// ---- M/N-contiguous operand (K x ext, row stride ld): tile columns origin .. origin + ROWS
template <int ROWS, int NW>
static void case_mncontig(bool kgather) {
    const int ext = rnd(1, 90) * 8, K = rnd(1, 700), ld = ext + rnd(0, 4) * 8;
    const int origin = rnd(0, (ext - 1) / ROWS) * ROWS;
    const int src_rows = kgather ? rnd(1, 900) : K;
    snprintf(g_case, sizeof g_case, "M/N-contiguous %dx%d waves %d ext %d origin %d K %d ld %d k-gathered %d", 64, ROWS, NW, ext,
             origin, K, ld, (int)kgather);
    GuardedMap map(K);
    for (int i = 0; i < K; ++i) map.data[i] = rnd(0, 9) == 0 ? rnd(-5, src_rows + 5) : rnd(0, src_rows - 1);
    OperandView<bf16> op{FAKE, ld, ext, origin};
    allow(0, FAKE, (int64_t)(src_rows - 1) * ld + ext);
    allow(1, nullptr, 0);
    if (kgather) {
        op.k_map = map.data; op.k_ext = K; op.map_rows = src_rows;
        drive64<TileLoaderKG<bf16, ROWS, NW>, true>(op, K, NW, ROWS);
    } else {
        drive64<TileLoader<bf16, ROWS, NW, true, false>, false>(op, K, NW, ROWS);
        if (NW == 4 && K % 32 == 0) drive32<Tile32Loader<bf16, ROWS, NW, true, false>>(op, K, NW, ROWS);
    }
    drive_tail<ROWS, NW * 64, true>(op, K);
}

// ---- an expert without rows whose (empty) map is the end of the map buffer
static void case_empty_group() {
    snprintf(g_case, sizeof g_case, "k-gathered loader of an expert without rows at the end of the map");
    GuardedMap map(1);
    OperandView<bf16> op{FAKE, 256, 256, 0};
    op.k_map = map.data + 1;          // row0 == total rows: nothing behind it may be read
    op.k_ext = 0;
    op.map_rows = 64;
    allow(0, FAKE, 64 * 256);
    for (int wave = 0; wave < 8; ++wave)
        for (int lane = 0; lane < 64; ++lane) {
            TileLoaderKG<bf16, 256, 8> l;
            l.init(op, wave, lane);
            l.fetch();
            l.prepare();
            g_sink += l.roff[0];      // the entries are used: the reads cannot be optimised away
        }
}

int main(int argc, char** argv) {
    const int reps = argc > 1 ? atoi(argv[1]) : 40;
    for (int i = 0; i < reps; ++i) {
        case_kcontig<256, 8>(false, false);
        case_kcontig<256, 8>(true, false);
        case_kcontig<256, 8>(false, true);
        case_kcontig<128, 4>(false, false);
        case_kcontig<128, 4>(true, false);
        case_kcontig<256, 4>(false, true);
        case_kcontig<128, 8>(false, false);
        case_mncontig<256, 8>(false);
        case_mncontig<256, 8>(true);
        case_mncontig<128, 4>(false);
        case_mncontig<256, 4>(false);
        case_mncontig<128, 8>(true);
    }
    case_empty_group();
    printf("requests %ld bad %ld\n", g_requests, g_bad);
    return g_bad ? 1 : 0;
}
"""


def _lifted_source():
    core = open(os.path.join(CSRC, "gemm_core.h")).read()
    core2 = open(os.path.join(CSRC, "gemm_core2.h")).read()
    parts = [
        _block(core, r"^template <typename T>\nstruct OperandView \{"),
        _line(core2, "FX_DEV int swz(int r)"),
        _line(core2, "FX_DEV int swz_tr(int k)"),
        _line(core2, "FX_DEV int swz_k(int r)"),
        _block(core2, r"^template <int ROWS, int NT>\nstruct Staged2 \{"),
        _block(core2, r"^template <typename T, int ROWS, int NT, bool MN_CONTIG>\nFX_DEV void stage2_load\("),
        _block(core2, r"^template <typename T, int ROWS, int NW, bool MN, bool DUAL>\nstruct TileLoader \{"),
        _block(core2, r"^template <typename T, int ROWS, int NW>\nstruct TileLoaderKG \{"),
        _block(core2, r"^template <typename T, int ROWS, int NW, bool MN, bool DUAL>\nstruct Tile32Loader \{"),
    ]
    return "\n\n".join(parts)


def test_every_request_of_the_tile_loaders_stays_inside_its_operand(tmp_path):
    src = tmp_path / "loader_audit.cpp"
    exe = tmp_path / "loader_audit"
    src.write_text(HARNESS.replace("@@LIFTED@@", _lifted_source()))
    build = subprocess.run(["g++", "-std=c++17", "-O1", "-Wno-attributes", "-o", str(exe), str(src)], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-4000:]
    run = subprocess.run([str(exe), "200"], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, f"rc {run.returncode}\n{run.stdout[-2000:]}\n{run.stderr[-4000:]}"
    requests = int(re.search(r"requests (\d+) bad 0", run.stdout).group(1))
    assert requests > 10_000_000       # the sweep really went through the K loops
