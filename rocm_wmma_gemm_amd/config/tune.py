#!/usr/bin/env python3
"""Offline tuner for the gfx950 GEMM library.

For each requested shape, layout triple and type pair it searches the kernel-config
space -- pipeline, workgroup tile (block_m, block_n, block_k), wave grid, band height of
the tile walk, split-K form, line touches ahead of the loads -- times candidates on the GPU through the library's tuner
hook and writes the winners as gemm_config_gfx950_f16.json / _f32.json in the schema the
config generator reads.

Role of the reference's config/tune.py + config/tuner.cpp (reference
rocm_wmma_gemm/config/tune.py:75-140 parameter space and constraints, :442-690 the GOMEA
search, :692-765,848-933 the driver; config/tuner.cpp:237-454 compile one tuple at run
time and time it):
  * the space is open: a tuple that is not among the library's compiled variants
    (csrc/variants.def) is compiled at tune time from csrc/kernel_jit.hip into a small
    library of its own (hipcc, a few seconds) and registered with the loaded GEMM library
    (rocm_wmma_gemm_register_variant), after which it runs through the same host path --
    split-K, reduce, padded copies -- as a compiled variant;
  * --search gomea walks that space with a linkage-tree GOMEA (population, linkage tree
    from mutual information by UPGMA, gene-pool optimal mixing, forced improvement towards
    the best solution, interleaved populations of doubling size), the reference's search;
    --search exhaustive times every compiled variant x band height x split instead, which
    is affordable for the short variant list and is what the shipped tables were made with;
  * kept from the reference's tool: the JSON schema (tune.py:905-913), one entry per
    (M, N, K, layout triple), --input to resume from / extend an existing file with
    untouched entries preserved (tune.py:772-822), --overwrite (tune.py:874), timing by GPU
    events around the enqueue;
  * every entry records the type pair it was timed on ("timed_on"); --type picks the pair,
    so bf16 shapes are tuned with bf16 kernels.
A winner that the library does not hold is written to the JSON like any other; --adopt
appends such tuples to csrc/variants.def so that the next build compiles them in (the
config generator refuses entries whose variant is not compiled).

Run on a machine with an MI355X:
    python rocm_wmma_gemm_amd/config/tune.py --type f32_bf16 --search gomea \\
        --shapes 8192,8192,8192 --layouts rcr --adopt
"""
from __future__ import annotations

import argparse
import ctypes
import hashlib
import json
import math
import os
import random
import subprocess
import sys
from dataclasses import dataclass

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.normpath(os.path.join(HERE, "..", ".."))
CSRC = os.path.normpath(os.path.join(HERE, "..", "csrc"))
sys.path.insert(0, ROOT)

LAYOUT_NAME = {0: "row_major", 1: "col_major"}
TYPE_PAIRS = ("f16_f16", "f32_f16", "bf16_bf16", "f32_bf16")  # index = the library's type_idx
CUS = 256  # compute units of an MI355X
DEFAULT_SHAPES = [
    # the reference's tuned sizes (gemm_config_gfx1100_f16.json)
    (1024, 1024, 1024), (2048, 2048, 2048), (2048, 5120, 5120), (4096, 2048, 64),
    (4096, 4096, 1024), (4096, 4096, 4096), (4096, 4096, 16384), (4096, 5120, 5120),
    (4096, 16384, 4096), (8192, 4096, 128), (8192, 8192, 1024), (8192, 8192, 8192),
    (32768, 4096, 4096), (65536, 2048, 2048),
    # projection, decode-like, ragged and long-K shapes
    (8192, 4096, 2048), (4096, 14336, 4096), (16, 8192, 8192), (64, 8192, 8192),
    (128, 8192, 8192), (4095, 5121, 3001), (1000, 1000, 1000), (1024, 1024, 65536),
    # small shapes of the parity suite
    (128, 128, 128), (256, 256, 256), (512, 512, 512),
    # square sizes whose tile count does not divide by the CU count
    (1536, 1536, 1536), (3072, 3072, 3072), (6144, 6144, 6144),
    # transformer projection shapes (hidden 4096 / 8192, feed-forward 11008 / 14336 / 28672)
    (4096, 11008, 4096), (4096, 4096, 11008), (8192, 8192, 4096), (4096, 12288, 4096),
    (8192, 1024, 8192), (4096, 4096, 14336), (2048, 8192, 2048), (12288, 4096, 4096),
    (5120, 5120, 5120), (8192, 3584, 7168), (7168, 7168, 7168), (8192, 28672, 8192),
    (8192, 8192, 28672),
]


def parse_shapes(text: str):
    out = []
    for tok in text.split(":"):
        m, n, k = (int(x) for x in tok.split(","))
        out.append((m, n, k))
    return out


def key_of(entry: dict):
    r, lay = entry["range"], entry["layout"]
    return (r["M"], r["N"], r["K"], lay["A"], lay["B"], lay["C"])


# ----------------------------------------------------------------------------- the space
@dataclass(frozen=True)
class Tile:
    """A kernel tuple: what csrc/variants.def lists per line."""
    block_m: int
    block_n: int
    block_k: int
    warps_m: int
    warps_n: int
    pipeline: int

    # (32 x 32 MFMA tiles per wave; 0.5 for a 16-wide side of the whole-K streaming kernel's tile)
    @property
    def warp_tile_m(self):
        return self.block_m // self.warps_m // 32 if self.block_m % (32 * self.warps_m) == 0 else 0.5

    @property
    def warp_tile_n(self):
        return self.block_n // self.warps_n // 32 if self.block_n % (32 * self.warps_n) == 0 else 0.5


# Genes of the search (reference tune.py:75-82 has warps_m, warps_n, warp_tile_m, warp_tile_n,
# swizzle, bits; here the tile is spelled by its extents, and K-step, pipeline and split-K
# form are genes too).
GENES = {
    "pipeline": [0, 1, 2, 3, 4, 5, 6],
    "block_m": [16, 32, 64, 128, 192, 256],
    "block_n": [16, 32, 64, 128, 192, 256],
    "block_k": [32, 64],
    "waves": [(1, 2), (2, 1), (1, 4), (4, 1), (2, 2), (2, 4), (4, 2)],
    "swizzle": [1, 4, 8, 16, -4, -8],
    "split": [1, 2, 4, 8, 16, 32, -1, -2, -3, -4, -6, -8],
    # the plan's fourth field: line touches one K tile ahead (1), K tiles in runs of 8 with the
    # XCDs out of step (64 = code 4 in bits 4-7), workgroups that start each group of 4 or 8
    # K tiles at different tiles (0x200, 0x300 = codes 2, 3 in bits 8-9)
    "touch": [0, 1, 64, 0x200, 0x300],
}
GENE_ORDER = list(GENES)


def kernel_space_layout(la: int, lb: int, lc: int):
    """(rows-operand K-contiguous, columns-operand K-contiguous) as the kernels see the
    problem: they write a row-major C, a column-major C runs as the transposed problem."""
    a_k, b_k = la == 0, lb == 1
    return (b_k, a_k) if lc == 1 else (a_k, b_k)


def ring_stages(t: Tile) -> int:
    return 4 if t.pipeline == 6 or (t.pipeline != 0 and t.block_k == 32) else 2


def tile_feasible(t: Tile, a_kmajor: bool, b_kmajor: bool) -> bool:
    """What the kernel templates take (their static_asserts, restated so that the search
    does not spend a compile on a tuple that cannot build; reference tune.py:105-140)."""
    waves = t.warps_m * t.warps_n
    if t.pipeline == 7:
        # whole-K streaming kernel: small tiles (at most one side 16 wide), stages of 128,
        # either layout of an operand
        return (t.block_k == 128 and t.block_m in (16, 32, 64, 128) and t.block_n in (16, 32, 64, 128)
                and 48 <= t.block_m + t.block_n <= 192
                and (t.warps_m, t.warps_n) == (max(1, t.block_m // 32), max(1, t.block_n // 32)))
    if t.block_m % (32 * t.warps_m) or t.block_n % (32 * t.warps_n):
        return False
    if t.block_k == 128:
        return False
    wtm, wtn = t.block_m // t.warps_m, t.block_n // t.warps_n
    if wtm * wtn // 64 > 256:  # accumulator registers per lane
        return False
    stages = ring_stages(t)
    if stages * (t.block_m + t.block_n) * t.block_k * 2 > 160 * 1024:
        return False
    if t.pipeline == 0:
        # register-staged loads: every 16-byte piece of a tile belongs to one thread
        threads = 64 * waves
        return all((rows * t.block_k // 8) % threads == 0 for rows in (t.block_m, t.block_n))
    # direct-to-LDS pipelines: 1 KiB per load instruction, dealt over the waves
    for rows, kmajor in ((t.block_m, a_kmajor), (t.block_n, b_kmajor)):
        loads = rows * t.block_k * 2 // 1024
        if loads == 0 or loads % waves or (rows * t.block_k * 2) % 1024:
            return False
        if not kmajor and rows % 128:
            return False
    per_wave = (t.block_m + t.block_n) * t.block_k * 2 // 1024 // waves
    if (stages - 1) * per_wave >= 64:
        return False
    if t.pipeline in (2, 4):
        return waves == 8
    if t.pipeline in (3, 6):
        return t.block_k == 64
    if t.pipeline == 5:
        return (t.warps_m, t.warps_n) == (2, 2) and t.block_k in (32, 64) and t.block_m in (192, 256) \
            and t.block_n in (192, 256)
    return True


def split_feasible(t: Tile, swizzle: int, split: int, rows: int, cols: int, K: int) -> bool:
    tiles = -(-rows // t.block_m) * -(-cols // t.block_n)
    k_steps = -(-K // t.block_k)
    if (t.block_m >= 192 and rows < 192) or (t.block_n >= 192 and cols < 192):
        return False  # a tile much larger than the problem only wastes work
    if tiles <= 8 and swizzle != 1:
        return False
    if t.pipeline == 7:
        # a workgroup per tile over the whole K, or 2, 4 or 8 that share a tile and add their
        # parts up inside the launch (whole stages of 128 each, at least two, the last of K may
        # be cut short; a counter per tile):
        # no band height; worth a try when a 256 x 256 tiling leaves most compute units
        # without a tile
        stages = -(-K // 128)
        return swizzle == (1 if tiles <= 8 else 4) and K >= 128 and K % 8 == 0 \
            and -(-rows // 256) * -(-cols // 256) < CUS // 2 \
            and (split == 1 or (split in (2, 4, 8) and stages % split == 0 and stages // split >= 2
                                and tiles <= 4096 and tiles * split <= 4 * CUS))
    if split == 1:
        return True
    if split > 1:
        return tiles < CUS and k_steps >= 16 and tiles * split <= 2048 and k_steps // split >= 4
    if split == -1:
        return t.pipeline == 5 and tiles % CUS != 0 and tiles * k_steps >= 4 * CUS
    tail = tiles % CUS
    return (tiles > CUS and 0 < tail <= CUS * 3 // 4 and k_steps >= 16
            and tail * -split <= CUS * 5 // 4 and k_steps // -split >= 4)


def touch_feasible(t: Tile, touch: int, K: int) -> bool:
    """Line touches are the persistent kernel's, and only worth a try on a long K."""
    return touch == 0 or (t.pipeline == 5 and K >= 8192)


def k_run_of(touch: int) -> int:
    code = (touch >> 4) & 15
    return 0 if code == 0 else 1 << (code - 1)


def k_group_of(touch: int) -> int:
    code = (touch >> 8) & 3
    return 0 if code == 0 else 1 << code


def touch_field_of(cfg: dict) -> int:
    group = int(cfg.get("k_group", 0))
    return ((cfg.get("touch_ahead", 0) & 15) | (int(cfg.get("k_runs", 0)).bit_length() << 4)
            | ((group.bit_length() - 1 if group else 0) << 8))


def decode(genes: tuple) -> tuple:
    """(tile, swizzle, split, touch) of a gene tuple."""
    g = dict(zip(GENE_ORDER, genes))
    wm, wn = g["waves"]
    return (Tile(g["block_m"], g["block_n"], g["block_k"], wm, wn, g["pipeline"]), g["swizzle"], g["split"],
            g["touch"])


def encode(t: Tile, swizzle: int, split: int, touch: int = 0):
    """Genes of a (tile, swizzle, split, touch) tuple, or None if a value is outside the domains."""
    values = dict(pipeline=t.pipeline, block_m=t.block_m, block_n=t.block_n, block_k=t.block_k,
                  waves=(t.warps_m, t.warps_n), swizzle=swizzle, split=split, touch=touch)
    if any(values[g] not in GENES[g] for g in GENE_ORDER):
        return None
    return tuple(values[g] for g in GENE_ORDER)


def tuple_of(cfg: dict):
    """(tile, swizzle, split, touch) of a JSON "config" object."""
    t = Tile(int(cfg["warps_m"] * cfg["warp_tile_m"] * 32), int(cfg["warps_n"] * cfg["warp_tile_n"] * 32),
             cfg.get("block_k", 64), cfg["warps_m"], cfg["warps_n"], cfg.get("pipeline", 0))
    split = -1 if cfg.get("stream_k") else (-cfg["tail_split"] if cfg.get("tail_split", 0) > 1
                                            else cfg.get("split_k", 1))
    return t, cfg.get("swizzle", 4), split, touch_field_of(cfg)


def config_json(t, swizzle: int, split_k: int, touch: int = 0) -> dict:
    """split_k as the library's hook takes it: s > 1 every tile split, -s (s > 1) only the
    tail wave, -1 the persistent kernel's walk by K tile."""
    cfg = {"warps_m": t.warps_m, "warps_n": t.warps_n, "warp_tile_m": t.warp_tile_m,
           "warp_tile_n": t.warp_tile_n, "swizzle": swizzle, "bits": 128,
           "block_k": t.block_k, "pipeline": t.pipeline, "split_k": max(split_k, 1)}
    if split_k < -1:
        cfg["tail_split"] = -split_k
    if split_k == -1:
        cfg["stream_k"] = 1
    if touch & 15:
        cfg["touch_ahead"] = touch & 15
    if k_run_of(touch):
        cfg["k_runs"] = k_run_of(touch)
    if k_group_of(touch):
        cfg["k_group"] = k_group_of(touch)
    return cfg


# ----------------------------------------------------------------------------- GOMEA
def _mutual_information(pop, i, j):
    n = len(pop)
    ci, cj, cij = {}, {}, {}
    for x in pop:
        ci[x[i]] = ci.get(x[i], 0) + 1
        cj[x[j]] = cj.get(x[j], 0) + 1
        cij[(x[i], x[j])] = cij.get((x[i], x[j]), 0) + 1
    return sum(c / n * math.log(c * n / (ci[a] * cj[b])) for (a, b), c in cij.items())


def linkage_tree(pop, n_genes):
    """Family of subsets by UPGMA on mutual information between genes (reference
    tune.py:520-590): singletons first, then each merge; the root (all genes) is left out."""
    clusters = [[g] for g in range(n_genes)]
    mi = {(i, j): _mutual_information(pop, i, j) for i in range(n_genes) for j in range(i + 1, n_genes)}
    fos = [list(c) for c in clusters]

    def similarity(a, b):
        return sum(mi[(min(i, j), max(i, j))] for i in a for j in b) / (len(a) * len(b))

    while len(clusters) > 2:
        best = max(((similarity(a, b), ia, ib) for ia, a in enumerate(clusters)
                    for ib, b in enumerate(clusters) if ia < ib), key=lambda t: t[0])
        _, ia, ib = best
        merged = clusters[ia] + clusters[ib]
        clusters = [c for k, c in enumerate(clusters) if k not in (ia, ib)] + [merged]
        fos.append(merged)
    return fos


def gomea(domains, feasible, evaluate, budget, rng, first_population=8, seeds=(), log=None, stats=None):
    """Minimises evaluate(genes) over the product of `domains` (a list of value lists)
    restricted to feasible(genes).  evaluate returns a time, or None for a candidate that
    turned out not to run (failed compile, kernel not built for the layout).  At most
    `budget` distinct candidates are evaluated.  `seeds` are known solutions (the compiled
    variants, a previous table's entry: the reference reloads prior results as baselines,
    tune.py:772-796) that join every population.  Returns (best genes, best time, evaluations).

    Interleaved multistart: populations of size 8, 16, 32, ... take generations in turn, a
    smaller one four times as often as the next larger (reference tune.py:600-690)."""
    n = len(domains)
    cache = {}

    def cost(x):
        if x not in cache:
            if len(cache) >= budget:
                return None
            t = evaluate(x)
            cache[x] = math.inf if t is None else t
            if log:
                log(x, cache[x])
        return cache[x]

    def random_solution():
        for _ in range(2000):
            x = tuple(rng.choice(d) for d in domains)
            if feasible(x):
                return x
        return None

    best = [None, math.inf]

    def note(x, c):
        if c is not None and c < best[1]:
            best[0], best[1] = x, c

    def new_population(size):
        pop = []
        for x in seeds:
            if feasible(x) and x not in pop:
                c = cost(x)
                if c is None:
                    break
                note(x, c)
                if math.isfinite(c):
                    pop.append(x)
        size = max(size, len(pop) + size // 2)  # room for random members beside the seeds
        for _ in range(size * 20):
            if len(pop) == size:
                break
            x = random_solution()
            if x is None or x in pop:
                continue
            c = cost(x)
            if c is None:
                break
            note(x, c)
            pop.append(x)
        return pop

    def mix(x, cx, donor, subset):
        if all(donor[g] == x[g] for g in subset):
            return x, cx, False
        y = tuple(donor[g] if g in subset else x[g] for g in range(n))
        if not feasible(y):
            return x, cx, False
        cy = cost(y)
        if cy is None:
            return x, cx, False
        note(y, cy)
        if cy <= cx and y != x:
            return y, cy, cy < cx
        return x, cx, False

    def generation(pop):
        if len(pop) < 2:
            return pop
        fos = linkage_tree(pop, n)
        out = []
        for x in pop:
            cx = cost(x)
            if cx is None:
                out.append(x)
                continue
            improved = False
            for subset in rng.sample(fos, len(fos)):
                x, cx, better = mix(x, cx, rng.choice(pop), subset)
                improved = improved or better
            if not improved and best[0] is not None and best[0] != x:
                # forced improvement: mix with the best solution until something gets better
                for subset in rng.sample(fos, len(fos)):
                    x, cx, better = mix(x, cx, best[0], subset)
                    if better:
                        break
                else:
                    x, cx = best[0], best[1]
            out.append(x)
        return diversify(out)

    refills = [0]  # candidates timed only to refill a population (they do not count as progress)

    def diversify(pop):
        """Forced improvement turns members into copies of the best solution, and a
        population of copies teaches the next linkage tree nothing.  When fewer than half of
        the members are distinct, up to a quarter of them (copies only) are replaced by fresh
        random solutions.  (The reference keeps its populations apart with a niching hall of
        fame, tune.py:186-240; with 7 genes this is enough.)"""
        if len(set(pop)) * 2 >= len(pop):
            return pop
        seen, out, quota = set(), [], max(1, len(pop) // 4)
        for x in pop:
            if x in seen and quota > 0:
                y = random_solution()
                if y is not None and y not in seen and y not in pop:
                    known = y in cache
                    c = cost(y)
                    if c is not None:
                        refills[0] += 0 if known else 1
                        note(y, c)
                        if math.isfinite(c):
                            quota -= 1
                            seen.add(y)
                            out.append(y)
                            continue
            seen.add(x)
            out.append(x)
        return out

    def polish():
        """Every single-gene change of the best solution, until none improves it."""
        improved = True
        while improved and best[0] is not None and len(cache) < budget:
            improved = False
            for g in range(n):
                for value in domains[g]:
                    y = best[0][:g] + (value,) + best[0][g + 1:]
                    if y == best[0] or not feasible(y):
                        continue
                    before = best[1]
                    c = cost(y)
                    if c is None:
                        return
                    note(y, c)
                    improved = improved or best[1] < before

    populations, size, tick, stalls = [], first_population, 0, 0
    while len(cache) < budget and stalls < 3:
        before = len(cache) - refills[0]
        if not populations or tick % (4 ** len(populations)) == 0 or stalls:
            pop = new_population(size)
            if pop:
                populations.append(pop)
            size *= 2
        for level, pop in enumerate(populations):
            if tick % (4 ** level) == 0:
                populations[level] = generation(pop)
        tick += 1
        # a round that timed nothing new: the populations have converged; the next round
        # starts a larger one at once, and three such rounds in a row end the search
        stalls = stalls + 1 if len(cache) - refills[0] == before else 0
        if stalls == 1:
            polish()
    polish()
    if stats is not None:
        stats["refills"] = refills[0]  # candidates timed to replace copies in a population
    return best[0], best[1], len(cache)


# ----------------------------------------------------------------------------- run-time compile
class JitBuilder:
    """Compiles csrc/kernel_jit.hip for one tuple, type pair and pair of kernel-space operand
    layouts, loads the result and registers it with the GEMM library."""

    HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

    def __init__(self, lib, cache_dir=None):
        self._lib = lib  # ctypes handle of librocm_wmma_gemm_gfx950.so
        self.cache_dir = cache_dir or os.path.join(ROOT, "rocm_wmma_gemm_amd", "build", "jit")
        os.makedirs(self.cache_dir, exist_ok=True)
        self._loaded = {}   # (tile, type, ak, bk) -> variant index or None
        self._handles = []  # the libraries must stay loaded
        lib.rocm_wmma_gemm_register_variant.restype = ctypes.c_int
        lib.rocm_wmma_gemm_register_variant.argtypes = [ctypes.c_int] * 9 + [ctypes.c_void_p]

    def command(self, t: Tile, type_idx: int, ak: bool, bk: bool, out: str):
        return [self.HIPCC, "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
                "-packed-fp32-ops", "-O3", "-std=c++17", "-fPIC", "-shared",
                "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
                f"-DRWG_TYPE={type_idx}", f"-DRWG_AK={int(ak)}", f"-DRWG_BK={int(bk)}",
                f"-DRWG_JIT_BM={t.block_m}", f"-DRWG_JIT_BN={t.block_n}", f"-DRWG_JIT_BK={t.block_k}",
                f"-DRWG_JIT_WM={t.warps_m}", f"-DRWG_JIT_WN={t.warps_n}", f"-DRWG_JIT_PIPE={t.pipeline}",
                os.path.join(CSRC, "kernel_jit.hip"), "-o", out]

    def build(self, t: Tile, type_idx: int, ak: bool, bk: bool):
        """Path of the compiled library, or None if the tuple does not compile."""
        tag = f"{t.pipeline}_{t.block_m}x{t.block_n}x{t.block_k}_{t.warps_m}x{t.warps_n}_t{type_idx}_{int(ak)}{int(bk)}"
        src_hash = hashlib.sha1()
        for root, _, files in sorted(os.walk(CSRC)):
            for f in sorted(files):
                if f.endswith((".hpp", ".hip", ".def")) and f != "config_generated.hpp":
                    src_hash.update(open(os.path.join(root, f), "rb").read())
        out = os.path.join(self.cache_dir, f"rwg_jit_{tag}_{src_hash.hexdigest()[:10]}.so")
        if os.path.exists(out):
            return out
        r = subprocess.run(self.command(t, type_idx, ak, bk, out), capture_output=True, text=True)
        if r.returncode != 0 or not os.path.exists(out):
            return None
        return out

    def variant_index(self, t: Tile, type_idx: int, ak: bool, bk: bool):
        """Index under which the loaded GEMM library runs this tuple, compiling and
        registering it if need be; None if it cannot be built."""
        key = (t, type_idx, ak, bk)
        if key not in self._loaded:
            path = self.build(t, type_idx, ak, bk)
            idx = None
            if path is not None:
                h = ctypes.CDLL(path, mode=os.RTLD_NOW | os.RTLD_LOCAL)
                kernels = (ctypes.c_void_p * 9).in_dll(h, "rwg_jit_kernels")  # (host::num_modes)
                rc = self._lib.rocm_wmma_gemm_register_variant(
                    t.block_m, t.block_n, t.block_k, t.warps_m, t.warps_n, t.pipeline, type_idx,
                    int(ak), int(bk), ctypes.cast(kernels, ctypes.c_void_p))
                if rc >= 0:
                    idx = rc
                    self._handles.append(h)
            self._loaded[key] = idx
        return self._loaded[key]


def variants_def_line(index: int, t: Tile) -> str:
    return (f"RWG_VARIANT({index}, {t.block_m}, {t.block_n}, {t.block_k}, {t.warps_m}, {t.warps_n}, "
            f"{t.pipeline})")


def adopt(tiles, path=None) -> list:
    """Appends tuples that csrc/variants.def does not list; returns the lines added."""
    import re

    path = path or os.path.join(CSRC, "variants.def")
    text = open(path).read()
    have = {tuple(int(x) for x in m.groups()[1:]) for m in
            re.finditer(r"^RWG_VARIANT\((\d+),\s*(\d+),\s*(\d+),\s*(\d+),\s*(\d+),\s*(\d+),\s*(\d+)\)", text, re.M)}
    index = len(have)
    added = []
    for t in tiles:
        sig = (t.block_m, t.block_n, t.block_k, t.warps_m, t.warps_n, t.pipeline)
        if sig in have:
            continue
        have.add(sig)
        added.append(variants_def_line(index, t))
        index += 1
    if added:
        with open(path, "a") as f:
            f.write("".join(line + "\n" for line in added))
    return added


# ----------------------------------------------------------------------------- timing
def candidates(variants, M, N, K, lc):
    """(variant, swizzle, split_k, touch) tuples of the exhaustive search over compiled variants."""
    rows, cols = (M, N) if lc == 0 else (N, M)
    out = []
    for v in variants:
        t = Tile(v.block_m, v.block_n, v.block_k, v.warps_m, v.warps_n, v.pipeline)
        tiles = -(-rows // v.block_m) * -(-cols // v.block_n)
        for sw in ([1] if tiles <= 8 else [4, 8, 16, -4, -8]):
            for sk in GENES["split"]:
                if split_feasible(t, sw, sk, rows, cols, K):
                    out.extend((v, sw, sk, touch) for touch in GENES["touch"] if touch_feasible(t, touch, K))
    return out


def time_candidate(L, torch, index, sw, sk, touch, C, A, B, M, N, K, lc, la, lb, reps, warmup):
    """Milliseconds per call of one plan, calls back to back (what a caller's loop sees:
    the launch of a call overlaps the call before it): the median of three runs of at least
    `reps` calls and 2 ms each."""
    for _ in range(warmup):
        rc = L.run_variant(index, sw, sk, C, A, B, M, N, K, lc, la, lb, touch_ahead=touch)
        if rc != 0:
            return None
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    runs = []
    while len(runs) < 3:
        start.record()
        for _ in range(reps):
            L.run_variant(index, sw, sk, C, A, B, M, N, K, lc, la, lb, touch_ahead=touch)
        stop.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(stop)
        if ms < 2.0 and reps < 1024:
            reps *= 4
            continue
        runs.append(ms / reps)
    return sorted(runs)[1]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--type", choices=TYPE_PAIRS, default=None,
                    help="type pair to time (C type _ A/B type); decides the output file: "
                         "16-bit C -> _f16.json, fp32 C -> _f32.json")
    ap.add_argument("--type-group", choices=["f16", "f32"], default=None,
                    help="older spelling: f16 = --type f16_f16, f32 = --type f32_f16")
    ap.add_argument("--search", choices=["exhaustive", "gomea"], default="exhaustive")
    ap.add_argument("--budget", type=int, default=120, help="gomea: candidates timed per entry")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--shapes", default=None, help="M,N,K:M,N,K:... (default: built-in list)")
    ap.add_argument("--layouts", default="all", help="comma list of A,B,C triples like rcr, or 'all'")
    ap.add_argument("--input", default=None, help="existing JSON to extend")
    ap.add_argument("--output", default=None)
    ap.add_argument("--overwrite", action="store_true", help="re-tune entries present in --input")
    ap.add_argument("--adopt", action="store_true",
                    help="append winning tuples the library does not hold to csrc/variants.def")
    ap.add_argument("--reps", type=int, default=15)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--log", default=None, help="write every timing to this file")
    a = ap.parse_args(argv)
    type_name = a.type or {"f16": "f16_f16", "f32": "f32_f16", None: "f16_f16"}[a.type_group]
    type_idx = TYPE_PAIRS.index(type_name)
    group = "f32" if type_name.startswith("f32") else "f16"

    import torch

    import rocm_wmma_gemm_amd as R

    L = R.Loader()
    compiled = L.variants()
    index_of = {Tile(v.block_m, v.block_n, v.block_k, v.warps_m, v.warps_n, v.pipeline): v.index
                for v in compiled}
    jit = JitBuilder(L._lib)
    out_path = a.output or os.path.join(HERE, f"gemm_config_{L.arch}_{group}.json")
    in_path = a.input or (out_path if os.path.exists(out_path) else None)
    table = {}
    if in_path and os.path.exists(in_path):
        for e in json.load(open(in_path))["configurations"]:
            table[key_of(e)] = e
    shapes = parse_shapes(a.shapes) if a.shapes else DEFAULT_SHAPES
    if a.layouts == "all":
        layouts = [(la, lb, lc) for la in (0, 1) for lb in (0, 1) for lc in (0, 1)]
    else:
        layouts = [tuple("rc".index(ch) for ch in tok) for tok in a.layouts.split(",")]
    in_dtype = torch.bfloat16 if "bf16" in type_name.split("_", 1)[1] else torch.float16
    c_dtype = torch.float32 if group == "f32" else in_dtype
    log = open(a.log, "w") if a.log else None
    rng = random.Random(a.seed)
    new_tiles = []

    for (M, N, K) in shapes:
        A = (torch.rand(M * K, device="cuda") * 2 - 1).to(in_dtype)
        B = (torch.rand(K * N, device="cuda") * 2 - 1).to(in_dtype)
        C = torch.empty(M * N, dtype=c_dtype, device="cuda")
        for (la, lb, lc) in layouts:
            key = (M, N, K, LAYOUT_NAME[la], LAYOUT_NAME[lb], LAYOUT_NAME[lc])
            if key in table and not a.overwrite:
                continue
            rows, cols = (M, N) if lc == 0 else (N, M)
            ak, bk = kernel_space_layout(la, lb, lc)
            lay = "rc"[la] + "rc"[lb] + "rc"[lc]

            def run(tile, sw, sk, touch=0):
                index = index_of.get(tile)
                if index is None:
                    index = jit.variant_index(tile, type_idx, ak, bk)
                    if index is None:
                        return None
                ms = time_candidate(L, torch, index, sw, sk, touch, C, A, B, M, N, K, lc, la, lb, a.reps,
                                    a.warmup)
                if log and ms is not None:
                    log.write(f"{M},{N},{K} {lay} {type_name} p{tile.pipeline} {tile.block_m}x{tile.block_n}x"
                              f"{tile.block_k} w{tile.warps_m}x{tile.warps_n} sw{sw} sk{sk} touch{touch} "
                              f"{'compiled' if tile in index_of else 'jit'} {ms:.4f} ms "
                              f"{2.0 * M * N * K / ms / 1e9:.1f} TFLOP/s\n")
                    log.flush()
                return ms

            best = None
            if a.search == "exhaustive":
                for (v, sw, sk, touch) in candidates(compiled, M, N, K, lc):
                    tile = Tile(v.block_m, v.block_n, v.block_k, v.warps_m, v.warps_n, v.pipeline)
                    ms = run(tile, sw, sk, touch)
                    if ms is not None and (best is None or ms < best[0]):
                        best = (ms, tile, sw, sk, touch)
            else:
                domains = [GENES[g] for g in GENE_ORDER]

                def feasible(genes):
                    tile, sw, sk, touch = decode(genes)
                    return (tile_feasible(tile, ak, bk) and split_feasible(tile, sw, sk, rows, cols, K)
                            and touch_feasible(tile, touch, K))

                seeds = [encode(t, 1 if -(-rows // t.block_m) * -(-cols // t.block_n) <= 8 else 8, 1)
                         for t in index_of]
                prior = table.get(key)
                if prior is not None:
                    seeds.append(encode(*tuple_of(prior["config"])))
                genes, ms, evals = gomea(domains, feasible, lambda g: run(*decode(g)), a.budget, rng,
                                         seeds=[g for g in seeds if g is not None])
                if genes is not None and math.isfinite(ms):
                    best = (ms,) + decode(genes)
                    print(f"  gomea: {evals} candidates timed", flush=True)
            if best is None:
                continue
            ms, tile, sw, sk, touch = best
            entry = {"range": {"M": M, "N": N, "K": K},
                     "layout": {"A": key[3], "B": key[4], "C": key[5]},
                     "config": config_json(tile, sw, sk, touch), "timed_on": type_name}
            table[key] = entry
            if tile not in index_of:
                new_tiles.append(tile)
            print(f"{M}x{N}x{K} A={key[3][:3]} B={key[4][:3]} C={key[5][:3]} {type_name}: "
                  f"{tile.block_m}x{tile.block_n}x{tile.block_k}, {tile.warps_m}x{tile.warps_n} waves, "
                  f"pipeline {tile.pipeline}{'' if tile in index_of else ' (not in the library yet)'}, "
                  f"swizzle {sw} split_k {sk} touch {touch}: {ms:.4f} ms, {2.0 * M * N * K / ms / 1e9:.1f} TFLOP/s",
                  flush=True)
        del A, B, C
        # write after every shape: an interrupted run resumes from here with --input
        doc = {"configurations": [table[k] for k in sorted(table)]}
        with open(out_path, "w") as f:
            json.dump(doc, f, indent=4)
    print(f"wrote {out_path}: {len(table)} entries")
    if new_tiles:
        if a.adopt:
            for line in adopt(new_tiles):
                print("added to csrc/variants.def:", line)
            print("rebuild the library (make -C rocm_wmma_gemm_amd/csrc) to compile them in")
        else:
            print("winners the library does not hold (pass --adopt to add them to csrc/variants.def):")
            for i, t in enumerate(dict.fromkeys(new_tiles)):
                print("  " + variants_def_line(len(compiled) + i, t))
    return 0


if __name__ == "__main__":
    sys.exit(main())
