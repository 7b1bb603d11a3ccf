"""Launch plans on the CPU: what the library would enqueue for a call, and whether it is sound.

The host side of the library -- argument checks, workspace layout, choice of kernels, grids --
is compiled as it is into a host-only *trace build* (``build.build_trace``) in which every
``launch_kernel`` call is written down instead of made: kernel with its template arguments, grid,
block, dynamic LDS, every argument field by field.  Tensors are stand-ins: address ranges of a
made-up address space (nothing is dereferenced).  On those records this module runs

  * checks that hold for any launch: grid and block within the hardware's limits, LDS within the
    160 KiB of a CU and within the limit the launcher asked for, every pointer inside the tensor
    or workspace it was cut from, strided extents inside their tensors;
  * per-kernel *models*: a second statement, lane by lane, of the index arithmetic of the device
    code -- which rows and columns a lane's loads and stores name, whether the buffer range check
    lets them through, where they land in LDS, how often the tile loop runs, what the vmcnt waits
    are -- with the assertions that every access that passes the range check is one the algorithm
    means (a row below N, a column below the width) and lies inside the tensor, that every access
    the algorithm means passes the range check, and that trip counts and barrier counts do not
    depend on the wave.

Used by tests/test_launch_plan_cpu.py.  Nothing here needs a GPU.
"""

from __future__ import annotations

import ctypes
import re
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np

from flashy_linear_attention_amd import _lib, build

LDS_PER_CU = 160 * 1024
K_OOB = 0x40000000
DEFAULT_LDS_LIMIT = 64 * 1024  # dynamic LDS a kernel may use without raising its limit

_trace_lib = None


def trace_lib(rebuild: bool = False) -> ctypes.CDLL:
    """The trace build of the library (built on first use)."""
    global _trace_lib
    if _trace_lib is None or rebuild:
        path = build.build_trace()
        lib = ctypes.CDLL(path)
        for name, (argtypes, restype) in _lib.SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
        lib.fla_trace_take.argtypes = [ctypes.c_char_p, ctypes.c_int64]
        lib.fla_trace_take.restype = ctypes.c_int64
        _trace_lib = lib
    return _trace_lib


# ---------------------------------------------------------------------------------------------
# a made-up address space

@dataclass
class Region:
    name: str
    lo: int
    hi: int


class Arena:
    """Hands out disjoint address ranges, 4 GiB apart or more, 256-byte aligned (plus `misalign`)."""

    def __init__(self):
        self.regions: List[Region] = []
        self._next = 1 << 40

    def alloc(self, name: str, nbytes: int, misalign: int = 0) -> int:
        lo = self._next + misalign
        self.regions.append(Region(name, lo, lo + nbytes))
        self._next += ((nbytes + (1 << 32)) >> 32) << 33
        return lo

    def find(self, addr: int) -> Optional[Region]:
        for r in self.regions:
            if r.lo <= addr < r.hi or (addr == r.lo == r.hi):
                return r
        return None

    def require(self, what: str, lo: int, hi: int) -> Region:
        """[lo, hi) must lie inside one region."""
        r = self.find(lo)
        assert r is not None, f"{what}: address {lo:#x} is in no tensor or workspace"
        assert hi <= r.hi, f"{what}: [{lo - r.lo}, {hi - r.lo}) runs past the end of {r.name} ({r.hi - r.lo} bytes)"
        return r


@dataclass
class Tensor:
    ptr: int
    strides: Tuple[int, int, int, int]
    shape: Tuple[int, int, int, int]

    def strides_arg(self):
        return (ctypes.c_int64 * 4)(*self.strides)


def make_tensor(arena: Arena, name: str, b: int, h: int, n: int, w: int, layout: str = "contiguous",
                misalign: int = 0) -> Tensor:
    """(B, H, N, W) 16-bit tensor: contiguous, stored as (B, N, H, W) ("bnhd"), with padded rows
    ("padded": row stride W + 8), with an odd row stride ("odd": W + 1, rows not 16-byte aligned), or
    expanded along the sequence ("expanded": one stored row per head, row stride 0)."""
    if layout == "contiguous":
        st = (h * n * w, n * w, w, 1)
    elif layout == "bnhd":
        st = (n * h * w, w, h * w, 1)
    elif layout == "padded":
        st = (h * n * (w + 8), n * (w + 8), w + 8, 1)
    elif layout == "odd":
        st = (h * n * (w + 1), n * (w + 1), w + 1, 1)
    elif layout == "expanded":  # one row, repeated along the sequence (stride 0)
        st = (h * w, w, 0, 1)
    else:
        raise ValueError(layout)
    last = (b - 1) * st[0] + (h - 1) * st[1] + (n - 1) * st[2] + w if min(b, h, n) > 0 else 0
    ptr = arena.alloc(name, 2 * last, misalign)
    return Tensor(ptr, st, (b, h, n, w))


# ---------------------------------------------------------------------------------------------
# records

@dataclass
class Launch:
    kernel: str            # base name, e.g. "tri_xyt_z_fast_kernel"
    targs: List            # template arguments: "bf16" / "f16", ints, bools
    grid: Tuple[int, int, int]
    block: int
    lds: int
    args: Dict[str, float]  # "a0.x" -> value
    lds_limit: int = DEFAULT_LDS_LIMIT

    def struct(self, prefix: str) -> Dict[str, float]:
        pre = prefix + "."
        return {k[len(pre):]: v for k, v in self.args.items() if k.startswith(pre)}


_TARG = re.compile(r"DF16b|DF16_|Li(\d+)E|Lin(\d+)E|Lb([01])E")


def _parse_symbol(sym: str) -> Tuple[str, List]:
    """("tri_xyt_z_fast_kernel", ["bf16", 128, 128, False, 1]) from the (mangled) host symbol."""
    m = re.match(r"_ZN3fla(\d+)", sym)
    if m:
        n = int(m.group(1))
        start = m.end()
        name = sym[start:start + n]
        rest = sym[start + n:]
        targs: List = []
        if rest.startswith("I"):
            body = rest[1:]
            pos = 0
            while pos < len(body):
                t = _TARG.match(body, pos)
                if not t:
                    break
                tok = t.group(0)
                if tok == "DF16b":
                    targs.append("bf16")
                elif tok == "DF16_":
                    targs.append("f16")
                elif tok.startswith("Lb"):
                    targs.append(tok[2] == "1")
                elif tok.startswith("Lin"):
                    targs.append(-int(t.group(2)))
                else:
                    targs.append(int(t.group(1)))
                pos = t.end()
        return name, targs
    m = re.search(r"\[Kern = &(?:[A-Za-z_()\s]+::)*([A-Za-z_][A-Za-z0-9_]*)\]", sym)
    if m:  # a kernel with internal linkage: the name only
        return m.group(1), []
    # demangled: "void fla::norm_scan_kernel<0>(float*, ...)", "void (anonymous namespace)::pack_pair_kernel<_Float16>(...)"
    m = re.match(r"(?:void )?(?:[A-Za-z_()\s]+::)*([A-Za-z_][A-Za-z0-9_]*)(?:<([^>]*)>)?\(", sym)
    if m:
        targs = []
        for tok in (m.group(2) or "").split(","):
            tok = tok.strip()
            if not tok:
                continue
            targs.append("bf16" if tok == "__bf16" else "f16" if tok == "_Float16" else tok == "true" if tok in ("true", "false")
                         else int(tok))
        return m.group(1), targs
    # mangled, outside namespace fla (the anonymous namespace of the C ABI's translation unit)
    m = re.search(r"_GLOBAL__N_1(\d+)", sym)
    assert m, f"unrecognised kernel symbol {sym}"
    n = int(m.group(1))
    name = sym[m.end():m.end() + n]
    targs = []
    for t in _TARG.finditer(sym[m.end() + n:]):
        tok = t.group(0)
        targs.append("bf16" if tok == "DF16b" else "f16" if tok == "DF16_" else (tok[2] == "1") if tok.startswith("Lb")
                     else int(t.group(1)))
    return name, targs


def take_launches(lib) -> List[Launch]:
    n = lib.fla_trace_take(None, 0)
    buf = ctypes.create_string_buffer(n)
    lib.fla_trace_take(buf, n)
    out: List[Launch] = []
    limits: Dict[str, int] = {}
    for line in buf.value.decode().splitlines():
        if not line:
            continue
        if line.startswith("lds_limit="):
            val, sym = line.split(";kernel=", 1)
            limits[sym] = max(limits.get(sym, 0), int(val[len("lds_limit="):]))
            continue
        parts = line.split(";")
        kv = dict(p.split("=", 1) for p in parts)
        sym = kv.pop("kernel")
        name, targs = _parse_symbol(sym)
        grid = tuple(int(x) for x in kv.pop("grid").split(","))
        block = int(kv.pop("block"))
        lds = int(kv.pop("lds"))
        args = {k: (float(v) if ("." in v or "e" in v or "n" in v) else int(v)) for k, v in kv.items()}
        out.append(Launch(name, targs, grid, block, lds, args, limits.get(sym, DEFAULT_LDS_LIMIT)))
    return out


# ---------------------------------------------------------------------------------------------
# checks that hold for any launch

def check_launch_limits(l: Launch) -> None:
    gx, gy, gz = l.grid
    assert 1 <= gx <= 0x7fffffff, f"{l.kernel}: grid.x = {gx}"
    assert 1 <= gy <= 65535 and 1 <= gz <= 65535, f"{l.kernel}: grid.y, z = {gy}, {gz}"
    assert l.block == 256, f"{l.kernel}: block = {l.block}"
    assert l.lds <= LDS_PER_CU, f"{l.kernel}: {l.lds} bytes of LDS"
    assert l.lds <= l.lds_limit, f"{l.kernel}: {l.lds} bytes of dynamic LDS, limit raised to {l.lds_limit} only"


def tensor_extent(p: Dict, ptr: str, sb: str, sh: str, sn: str, H: int, BH: int, N: int, width: int) -> Tuple[int, int]:
    """Byte range of a (B, H, N, width) tensor given by pointer and element strides in struct p."""
    B = BH // H
    lo = p[ptr]
    last = (B - 1) * p[sb] + (H - 1) * p[sh] + (N - 1) * p[sn] + width
    return lo, lo + 2 * last


# ---------------------------------------------------------------------------------------------
# model of the fast masked-product kernels (csrc/fla_tri_fast.h), quadratic walk

@dataclass
class FastCfg:
    DC: int
    DO: int
    chunked: bool
    MW: int = 0
    BM: int = 0
    BN: int = 64
    RY: int = 0
    RZ: int = 0
    CY: int = 0
    CZ: int = 0
    Y_BYTES: int = 0
    Z_BYTES: int = 0
    STAGE: int = 0
    NBUF: int = 0
    SMEM: int = 0
    STATE_BYTES: int = 0
    state_in_lds: bool = False
    min_waves: int = 1
    NIY: int = 0
    NIZ: int = 0
    NT: int = 0
    NYD: int = 0
    RO: int = 0
    supported: bool = False

    def __post_init__(self):
        DC, DO = self.DC, self.DO
        self.MW = 64 if DC // 2 + DO <= 192 else 32
        self.BM = 4 * self.MW
        self.RY, self.RZ = 2 * DC, 2 * DO
        self.CY, self.CZ = DC // 8, DO // 8
        self.Y_BYTES, self.Z_BYTES = 64 * self.RY, 64 * self.RZ
        self.STAGE = self.Y_BYTES + self.Z_BYTES
        max_slots = LDS_PER_CU // self.STAGE
        self.NBUF = self.BM // 64 if self.chunked else min(5, max_slots)
        self.SMEM = self.NBUF * self.STAGE
        self.supported = max_slots >= 3 and self.BM // 64 <= max_slots
        self.STATE_BYTES = ((DO + 63) // 64) * self.Y_BYTES
        self.state_in_lds = self.chunked and self.SMEM + self.STATE_BYTES <= LDS_PER_CU
        self.min_waves = 2 if DC <= 64 and DO <= 64 else 1
        self.NIY, self.NIZ = self.Y_BYTES // 4096, self.Z_BYTES // 4096
        self.NT = self.NIY + self.NIZ
        self.NYD = 1 if (4 * (1024 // self.RY)) % 16 == 0 else 2
        self.RO = 2 * DO + 16


def swizzle_y(CY: int, row):
    if CY == 4:
        return (row >> 2) & 3
    if CY == 8:
        return (row >> 1) & 7
    return row & 15


def swizzle_z(CZ: int, row):
    if CZ == 4:
        return ((row >> 1) & 1) << 1
    return (row & 3) << 1


def run_single_tiles(pairs: int, wg_per_cu: int) -> bool:
    return pairs < 256 * wg_per_cu and pairs % 256 != 0


@dataclass
class Stats:
    launches: int = 0
    workgroups: int = 0
    lane_accesses: int = 0
    kernels: Dict[str, int] = field(default_factory=dict)


def _buffer_check(what: str, offsets, meant, num_records: int, size: int = 16) -> None:
    """offsets: byte offsets into a raw buffer of num_records bytes; meant: which of them the algorithm
    means (a valid row and column).  The hardware returns zeros for offset + size > num_records."""
    offsets = np.asarray(offsets, dtype=np.int64)
    meant = np.asarray(meant, dtype=bool)
    assert (offsets >= 0).all() and (offsets < (1 << 32)).all(), f"{what}: offset outside 32 bits"
    passes = offsets + size <= num_records
    bad = passes & ~meant
    assert not bad.any(), f"{what}: {int(bad.sum())} accesses to rows or columns outside the problem pass the range check"
    bad = meant & ~passes
    assert not bad.any(), f"{what}: {int(bad.sum())} accesses the algorithm needs fail the range check"


def model_tri_fast(arena: Arena, l: Launch, p: Dict, T: str, DC: int, DO: int, chunked: bool, flags: int,
                   lds_expected: Optional[int], stats: Stats, max_heads: int = 3) -> None:
    """One product of a fast-path launch: p = the TriParams of this product."""
    cfg = FastCfg(DC, DO, chunked)
    assert cfg.supported
    N, BH, H = p["N"], p["BH"], p["H"]
    dc, dout = p["dc"], p["dout"]
    upper = p["upper"] != 0
    assert 1 <= dc <= DC and 1 <= dout <= DO and dc % 8 == 0 and dout % 8 == 0
    assert p["vec_x"] and p["vec_y"] and p["vec_z"] and p["vec_out"], "fast path launched on unaligned operands"
    for ptr in ("x", "y", "z", "out"):
        assert p[ptr] % 16 == 0
    for st in ("xs_b", "xs_h", "xs_n", "ys_b", "ys_h", "ys_n", "zs_b", "zs_h", "zs_n", "os_b", "os_h", "os_n"):
        assert p[st] % 8 == 0
    if lds_expected is not None:
        assert l.lds == lds_expected, f"{l.kernel}: {l.lds} bytes of LDS, the configuration needs {lds_expected}"
    # launcher's arithmetic
    n_tiles = -(-N // cfg.BM)
    assert p["n_tiles"] == n_tiles
    single = chunked or p["single"] != 0
    if not chunked:
        assert bool(p["single"]) == run_single_tiles(BH * ((n_tiles + 1) // 2), cfg.min_waves)
    n_pairs = n_tiles if single else (n_tiles + 1) // 2
    assert l.grid[0] == 8 * ((BH + 7) // 8) * n_pairs, f"{l.kernel}: grid.x = {l.grid[0]}"
    # vmcnt bookkeeping
    ahead = cfg.NBUF - 3 if cfg.NBUF > 3 else 0
    assert ahead * cfg.NT < 64, "wait_tile's vmcnt does not fit its 6-bit field"
    NIB = cfg.MW // 32
    KC = DC // 16
    # tensors
    xs2, ys2, zs2 = 2 * p["xs_n"], 2 * p["ys_n"], 2 * p["zs_n"]
    for nm, s2, w in (("x", xs2, dc), ("y", ys2, dc), ("z", zs2, dout)):
        assert N * s2 <= 0x3fffffff, f"{nm}: a (b, h) slice exceeds the 32-bit offsets"
    rec_x, rec_y, rec_z = (N - 1) * xs2 + dc * 2, (N - 1) * ys2 + dc * 2, (N - 1) * zs2 + dout * 2
    lanes = np.arange(64)
    l32, g = lanes & 31, lanes >> 5
    n_hl = (BH + 7) >> 3
    seen_tiles = set()
    # every workgroup index: its head and row tiles.  Heads differ in their base addresses only, so
    # the lane-level part runs for the first heads, the last one and every rank.
    sample_ranks = {0, 1, n_pairs // 2, n_pairs - 2, n_pairs - 1}
    for wg in range(l.grid[0]):
        xcd, slot = wg & 7, wg >> 3
        if single and not chunked:
            hl, rank = slot % n_hl, slot // n_hl
        else:
            hl, rank = slot // n_pairs, slot - (slot // n_pairs) * n_pairs
        bh = hl * 8 + xcd
        if bh >= BH:
            continue
        stats.workgroups += 1
        if chunked:
            tiles = [rank]
        elif single:
            tiles = [rank if upper else n_tiles - 1 - rank]
        else:
            tiles = [n_tiles - 1 - rank] + ([rank] if rank != n_tiles - 1 - rank else [])
        for t in tiles:
            assert 0 <= t < n_tiles
            assert (bh, t) not in seen_tiles, f"row tile {t} of head {bh} is computed twice"
            seen_tiles.add((bh, t))
        # lane level: the first and last heads (heads differ in their base addresses only), and the
        # ranks at both ends and in the middle (the others differ in the count of full tiles only)
        if bh not in (0, BH - 1) or rank not in sample_ranks:
            continue
        b, h = bh // H, bh % H
        X = p["x"] + 2 * (b * p["xs_b"] + h * p["xs_h"])
        Y = p["y"] + 2 * (b * p["ys_b"] + h * p["ys_h"])
        Z = p["z"] + 2 * (b * p["zs_b"] + h * p["zs_h"])
        O = p["out"] + 2 * (b * p["os_b"] + h * p["os_h"])
        # the buffer resources cover exactly this head's valid rows, inside the tensor
        arena.require("X rows", X, X + rec_x)
        arena.require("Y rows", Y, Y + rec_y)
        arena.require("Z rows", Z, Z + rec_z)
        ring0 = 0
        for pass_i, tile in enumerate(tiles):
            i0 = tile * cfg.BM
            assert i0 < N
            diag_rows = min(N - i0, cfg.BM)
            n_diag = -(-diag_rows // 64)
            if upper:
                rest = N - (i0 + cfg.BM)
                n_full = -(-rest // 64) if rest > 0 else 0
                full_row0 = i0 + cfg.BM
            else:
                n_full, full_row0 = i0 // 64, 0
            if chunked:
                n_full = 0
            n_seq = n_full + n_diag
            assert n_diag <= cfg.NBUF

            def tile_row0(q):
                return full_row0 + q * 64 if q < n_full else i0 + (q - n_full) * 64

            # ---- X fragments (per wave: rows of its row blocks; lane: row l32, columns 16 kc + 8 g)
            for wave in range(4):
                blks = [wave] + ([cfg.BM // 32 - 1 - wave] if NIB == 2 else [])
                for blk in blks:
                    row = i0 + blk * 32 + l32
                    for kc in range(KC):
                        col = kc * 16 + 8 * g
                        off = row * xs2 + col * 2 + np.where(col < dc, 0, K_OOB)
                        _buffer_check("X fragment load", off, (row < N) & (col < dc), rec_x)
                        stats.lane_accesses += 64
            # ---- the tile sequence as the kernel issues it: tiles 0 .. NBUF-2 up front, then tile
            # q + NBUF - 1 while tile q is consumed, for q < n_full; one more before the diagonal block
            issued = []  # (sequence index, ring slot byte offset)
            slot_of = lambda q: (ring0 + q * cfg.STAGE) % (cfg.NBUF * cfg.STAGE)
            if chunked:
                for q in range(cfg.BM // 64):
                    issued.append((q, q * cfg.STAGE))
            else:
                for q in range(cfg.NBUF - 1):
                    issued.append((q, slot_of(q)))
                for q in range(n_full):
                    issued.append((q + cfg.NBUF - 1, slot_of(q + cfg.NBUF - 1)))
                issued.append((n_full + cfg.NBUF - 1, slot_of(n_full + cfg.NBUF - 1)))
            # every tile the walk consumes has been issued, each into the slot the reads expect,
            # and a slot is not overwritten before its tile has been consumed
            first_issue = {}
            for order, (q, so) in enumerate(issued):
                first_issue.setdefault(q, (order, so))
            for q in range(n_seq):
                assert q in first_issue, f"tile {q} of the sequence is never requested"
                assert first_issue[q][1] == slot_of(q) if not chunked else True
            if not chunked:
                # tile q' goes into the slot of tile q' - NBUF: issued only after tile q' - NBUF + 1 began,
                # i.e. after the barrier that retires tile q' - NBUF
                for q, so in issued:
                    if q >= cfg.NBUF:
                        assert q - (cfg.NBUF - 1) >= 0
            # (lane level for the tiles at both ends of the sequence, around the diagonal block and past
            # the end; the tiles between are full tiles whose rows all lie below N)
            sample_q = {0, 1, n_full - 1, issued[-1][0]} | set(range(n_full, n_seq + 2))
            for q, so in issued:
                if q not in sample_q:
                    assert q > n_seq or (q < n_full and tile_row0(q) + 64 <= N)
                    continue
                exists = q < n_seq
                row0 = tile_row0(q) if exists else 0
                assert 0 <= so and so + cfg.STAGE <= cfg.SMEM
                for wave in range(4):
                    lds_wave = wave * 1024 + so
                    # Y loads
                    ystep = 4 * (1024 // cfg.RY)
                    for I in range(cfg.NIY):
                        v = I % cfg.NYD
                        row_l = v * ystep + wave * (1024 // cfg.RY) + lanes // cfg.CY
                        c = (lanes % cfg.CY) ^ swizzle_y(cfg.CY, row_l)
                        ydma = row_l * ys2 + c * 16 + np.where(c * 8 < dc, 0, K_OOB)
                        sbase = row0 * ys2 if exists else K_OOB
                        soff = sbase + (I - I % cfg.NYD) * ystep * ys2
                        off = ydma + soff
                        # where the bytes land, and which row / chunk of the tile the reads expect there
                        dst = lds_wave + I * 4096 + lanes * 16 - so
                        assert (dst >= 0).all() and (dst + 16 <= cfg.Y_BYTES).all()
                        lrow, lchunk = dst // cfg.RY, (dst % cfg.RY) // 16
                        want_chunk = lchunk ^ swizzle_y(cfg.CY, lrow)
                        grow = row0 + lrow
                        if exists:
                            want_off = grow * ys2 + want_chunk * 16
                            ok = (want_chunk * 8 < dc)
                            assert ((off == want_off) | ~ok).all(), "Y tile load: a lane fetches the wrong row or chunk"
                        _buffer_check("Y tile load", off, exists & (grow < N) & (want_chunk * 8 < dc), rec_y)
                        stats.lane_accesses += 64
                    zstep = 4 * (1024 // cfg.RZ)
                    for I in range(cfg.NIZ):
                        row_l = wave * (1024 // cfg.RZ) + lanes // cfg.CZ
                        c = (lanes % cfg.CZ) ^ swizzle_z(cfg.CZ, row_l)
                        zdma = row_l * zs2 + c * 16 + np.where(c * 8 < dout, 0, K_OOB)
                        sbase = row0 * zs2 if exists else K_OOB
                        off = zdma + sbase + I * zstep * zs2
                        dst = lds_wave + cfg.Y_BYTES + I * 4096 + lanes * 16 - so - cfg.Y_BYTES
                        assert (dst >= 0).all() and (dst + 16 <= cfg.Z_BYTES).all()
                        lrow, lchunk = dst // cfg.RZ, (dst % cfg.RZ) // 16
                        want_chunk = lchunk ^ swizzle_z(cfg.CZ, lrow)
                        grow = row0 + lrow
                        if exists:
                            want_off = grow * zs2 + want_chunk * 16
                            ok = (want_chunk * 8 < dout)
                            assert ((off == want_off) | ~ok).all(), "Z tile load: a lane fetches the wrong row or chunk"
                        _buffer_check("Z tile load", off, exists & (grow < N) & (want_chunk * 8 < dout), rec_z)
                        stats.lane_accesses += 64
            # ---- main loop trip count and barriers: workgroup-level scalars only (n_full), so every
            # wave passes the same barriers; the diagonal walk has none inside
            nsub = (diag_rows + 31) >> 5
            for wave in range(4):
                blks = [wave] + ([cfg.BM // 32 - 1 - wave] if NIB == 2 else [])
                s_lo = min(blks) if upper else 0
                s_hi = nsub - 1 if upper else min(max(blks), nsub - 1)
                for s8 in range(s_lo, s_hi + 1):
                    assert (s8 >> 1) < n_diag, "diagonal walk reads a tile that was not loaded"
            # ---- epilogue: rows out_i0 + r, 16-byte chunks cc of the output row
            CO = DO // 8
            tid = np.arange(256)
            for u in range(cfg.BM * CO // 256):
                c = tid + 256 * u
                r, cc = c // CO, c % CO
                row = i0 + r
                ok = (row < N) & (cc * 8 < dout)
                addr = O + 2 * (row * p["os_n"] + cc * 8)
                if ok.any():
                    arena.require("output store", int(addr[ok].min()), int(addr[ok].max()) + 16)
                    assert ((cc[ok] * 8 + 8) <= dout).all()
                stats.lane_accesses += 256
            assert cfg.BM * cfg.RO <= cfg.SMEM
            if flags & 1:  # the normaliser
                rows = i0 + np.arange(cfg.BM)
                rows = rows[rows < N]
                arena.require("denominator store", p["denom"] + 4 * (bh * N + int(rows.min())),
                              p["denom"] + 4 * (bh * N + int(rows.max())) + 4)
            # the second row tile's first requests go behind the epilogue's staging area
            stage_slots = -(-(cfg.BM * cfg.RO) // cfg.STAGE)
            if not chunked and cfg.NBUF - stage_slots >= 1 and cfg.NBUF >= 3:
                ring0 = stage_slots * cfg.STAGE
            else:
                ring0 = 0
    want = {(bh, t) for bh in range(BH) for t in range(n_tiles)}
    assert seen_tiles == want, f"{len(want - seen_tiles)} row tiles are computed by no workgroup"


# ---------------------------------------------------------------------------------------------
# model of the fused dV + dK kernel (csrc/fla_tri_pair.h)

def walk_swizzle(CR: int, row):
    if CR == 4:
        return (row >> 2) & 3
    if CR == 8:
        t = (row >> 1) & 7
        return ((t & 1) << 2) | (t >> 1)
    t = row & 15
    return ((t & 3) << 2) | (t >> 2)


def model_tri_pair(arena: Arena, l: Launch, p: Dict, D: int, stats: Stats) -> None:
    NIB = 2 if D <= 64 else 1
    BM = 4 * 32 * NIB
    RB, CR = 2 * D, D // 8
    TILE = 64 * RB
    STAGE = 2 * TILE
    NBUF = min(6, LDS_PER_CU // STAGE)
    NI = TILE // 4096
    NT, RPI = 2 * NI, 1024 // RB
    assert l.lds == NBUF * STAGE and BM // 64 <= NBUF - 1 and BM * (2 * D + 16) <= NBUF * STAGE
    assert (NBUF - 3) * NT < 64, "wait_tile's vmcnt does not fit its 6-bit field"
    assert NI == 1 or (4 * RPI) % 16 == 0
    N, BH, H, wa, wb = p["N"], p["BH"], p["H"], p["wa"], p["wb"]
    assert 1 <= wa <= D and 1 <= wb <= D and wa % 8 == 0 and wb % 8 == 0
    n_tiles = -(-N // BM)
    assert p["n_tiles"] == n_tiles
    single = p["single"] != 0
    assert single == run_single_tiles(BH * ((n_tiles + 1) // 2), 1)
    n_pairs = n_tiles if single else (n_tiles + 1) // 2
    assert l.grid == (8 * ((BH + 7) // 8) * n_pairs, 1, 1)
    for nm, ptr, sb, sh, sn, w in (("xa", "xa", "xas_b", "xas_h", "xas_n", wa), ("xb", "xb", "xbs_b", "xbs_h", "xbs_n", wb),
                                   ("ya", "ya", "yas_b", "yas_h", "yas_n", wa), ("yb", "yb", "ybs_b", "ybs_h", "ybs_n", wb),
                                   ("oa", "oa", "oas_b", "oas_h", "oas_n", wb), ("ob", "ob", "obs_b", "obs_h", "obs_n", wa)):
        lo, hi = tensor_extent(p, ptr, sb, sh, sn, H, BH, N, w)
        arena.require(f"fused dV + dK kernel, {nm}", lo, hi)
        assert p[ptr] % 16 == 0 and all(p[x] % 8 == 0 for x in (sb, sh, sn)) and p[sn] >= w
        assert N * p[sn] * 2 <= 0x3fffffff
    lanes = np.arange(64)
    seen = set()
    n_hl = (BH + 7) >> 3
    for wg in range(l.grid[0]):
        xcd, slot = wg & 7, wg >> 3
        hl, rank = (slot % n_hl, slot // n_hl) if single else (slot // n_pairs, slot % n_pairs)
        bh = hl * 8 + xcd
        if bh >= BH:
            continue
        stats.workgroups += 1
        tiles = [rank] if single or rank == n_tiles - 1 - rank else [rank, n_tiles - 1 - rank]
        for t in tiles:
            assert 0 <= t < n_tiles and (bh, t) not in seen
            seen.add((bh, t))
        if bh not in (0, BH - 1) or rank not in {0, 1, n_pairs // 2, n_pairs - 1}:
            continue
        for tile in tiles:
            i0 = tile * BM
            diag_rows = min(N - i0, BM)
            rest = N - (i0 + BM)
            n_full = -(-rest // 64) if rest > 0 else 0
            n_seq = n_full + -(-diag_rows // 64)
            for q in sorted({0, 1, n_full - 1, n_full + NBUF - 1} | set(range(n_full, n_seq + 2))):
                if q < 0:
                    continue
                exists = q < n_seq
                row0 = (i0 + BM + q * 64 if q < n_full else i0 + (q - n_full) * 64) if exists else 0
                for which, s2, w in ((0, 2 * p["yas_n"], wa), (1, 2 * p["ybs_n"], wb)):
                    rec = (N - 1) * s2 + w * 2
                    for wave in range(4):
                        row_l = wave * RPI + lanes // CR
                        c = (lanes % CR) ^ walk_swizzle(CR, row_l)
                        voff = row_l * s2 + c * 16 + np.where(c * 8 < w, 0, K_OOB)
                        for I in range(NI):
                            so = (row0 + I * 4 * RPI) * s2 if exists else K_OOB
                            dst = I * 4096 + wave * 1024 + lanes * 16  # within the operand's tile
                            lrow, lchunk = dst // RB, (dst % RB) // 16
                            want_chunk = lchunk ^ walk_swizzle(CR, lrow)
                            grow = row0 + lrow
                            if exists:
                                ok = want_chunk * 8 < w
                                assert ((voff + so == grow * s2 + want_chunk * 16) | ~ok).all(), \
                                    "fused kernel tile load: a lane fetches the wrong row or chunk"
                            _buffer_check("fused kernel tile load", voff + so, exists & (grow < N) & (want_chunk * 8 < w), rec)
                            stats.lane_accesses += 64
    assert seen == {(bh, t) for bh in range(BH) for t in range(n_tiles)}


# ---------------------------------------------------------------------------------------------
# model of the generic masked-product kernel (csrc/fla_tri_kernel.h)

def model_tri_generic(arena: Arena, l: Launch, p: Dict, DC: int, DO: int, stats: Stats) -> None:
    MW = 64 if DC // 2 + DO <= 192 else 32
    BM = 4 * MW
    N, BH, H = p["N"], p["BH"], p["H"]
    n_tiles = -(-N // BM)
    assert p["n_tiles"] == n_tiles and l.grid[0] == 8 * ((BH + 7) // 8) * n_tiles
    SY, SZ = DC * 2 + 16, DO * 2 + 64
    assert l.lds == 2 * 64 * (SY + SZ)
    assert 1 <= p["dc"] <= DC and 1 <= p["dout"] <= DO
    # element-wise bounds checks in the kernel: every access names a row < N and a column < width;
    # 16-byte accesses only with vec_* set
    for nm, ptr, sb, sh, sn, w, vec in (("x", "x", "xs_b", "xs_h", "xs_n", p["dc"], p["vec_x"]),
                                        ("y", "y", "ys_b", "ys_h", "ys_n", p["dc"], p["vec_y"]),
                                        ("z", "z", "zs_b", "zs_h", "zs_n", p["dout"], p["vec_z"]),
                                        ("out", "out", "os_b", "os_h", "os_n", p["dout"], p["vec_out"])):
        lo, hi = tensor_extent(p, ptr, sb, sh, sn, H, BH, N, w)
        arena.require(f"{nm} tensor", lo, hi)
        if vec:
            assert p[ptr] % 16 == 0 and w % 8 == 0 and all(p[s] % 8 == 0 for s in (sb, sh, sn))
    stats.workgroups += BH * n_tiles


# ---------------------------------------------------------------------------------------------
# models of the normaliser's passes (csrc/fla_norm.h)

def model_norm(arena: Arena, l: Launch, p: Dict, kernel: str, LPR: int, vec: bool, with_w: bool, stats: Stats) -> None:
    RPS = 64 // LPR
    NSEG = 4 * RPS
    R = NSEG * 16
    DP = LPR * 8
    N, BH, H, dqk, dv = p["N"], p["BH"], p["H"], p["dqk"], p["dv"]
    n_chunks = p["n_chunks"]
    assert n_chunks == -(-N // R), f"{kernel}: {n_chunks} chunks of {R} rows for N = {N}"
    assert l.grid[0] == n_chunks and l.grid[1] == BH
    tid = np.arange(256)
    lane, wave = tid & 63, tid >> 6
    li, seg = lane % LPR, wave * RPS + lane // LPR
    col = 8 * li

    def rows_access(what, ptr, sb, sh, sn, width, rows, cols, vecflag):
        """16-byte (or element-wise) accesses at (rows, cols) of a (B,H,N,width) tensor: all inside it."""
        ok = (rows < N) & (cols < width)
        if not ok.any():
            return
        if vecflag:
            assert width % 8 == 0 and p[ptr] % 16 == 0
        for bh in (0, BH - 1):
            b, h = bh // H, bh % H
            base = p[ptr] + 2 * (b * p[sb] + h * p[sh])
            addr = base + 2 * (rows[ok] * p[sn] + cols[ok])
            span = 16 if vecflag else 2 * np.minimum(8, width - cols[ok])
            arena.require(what, int(addr.min()), int((addr + span).max()))
        stats.lane_accesses += int(ok.sum())

    def scalar_access(what, ptr, index_lo, index_hi):
        arena.require(what, p[ptr] + 4 * index_lo, p[ptr] + 4 * index_hi + 4)

    for chunk in sorted({0, 1, n_chunks // 2, n_chunks - 2, n_chunks - 1} & set(range(n_chunks))):
        if kernel == "norm_bwd_pre_kernel":
            for r in range(16):
                row = (chunk * 16 + r) * NSEG + seg
                rows_access("g", "a", "as_b", "as_h", "as_n", dv, row, col, vec or p["vec_a"])
                rows_access("out", "b", "bs_b", "bs_h", "bs_n", dv, row, col, vec or p["vec_b"])
                rows_access("dO", "out", "os_b", "os_h", "os_n", dv, row, col, vec or p["vec_out"])
            continue
        row0 = chunk * R + seg * 16
        for r in range(16):
            row = row0 + r
            if kernel == "norm_chunk_sums_kernel":
                rows_access("k", "k", "ks_b", "ks_h", "ks_n", dqk, row, col, vec or p["vec_k"])
                if with_w:
                    rows_access("q", "q", "qs_b", "qs_h", "qs_n", dqk, row, col, vec or p["vec_q"])
            elif kernel == "norm_fwd_kernel":
                rows_access("k", "k", "ks_b", "ks_h", "ks_n", dqk, row, col, vec or p["vec_k"])
                rows_access("q", "q", "qs_b", "qs_h", "qs_n", dqk, row, col, vec or p["vec_q"])
                rows_access("O", "a", "as_b", "as_h", "as_n", dv, row, col, vec or p["vec_a"])
                rows_access("out", "out", "os_b", "os_h", "os_n", dv, row, col, vec or p["vec_out"])
            elif kernel == "norm_bwd_post_kernel":
                rows_access("k", "k", "ks_b", "ks_h", "ks_n", dqk, row, col, vec or p["vec_k"])
                rows_access("q", "q", "qs_b", "qs_h", "qs_n", dqk, row, col, vec or p["vec_q"])
                if not p["only_dk"]:
                    rows_access("dq", "dq", "dqs_b", "dqs_h", "dqs_n", dqk, row, col, vec or p["vec_dq"])
                rows_access("dk", "dk", "dks_b", "dks_h", "dks_n", dqk, row, col, vec or p["vec_dk"])
    # fp32 side buffers
    if kernel in ("norm_bwd_pre_kernel", "norm_fwd_kernel"):
        scalar_access("denom", "denom", 0, BH * N - 1)
    if kernel in ("norm_bwd_pre_kernel", "norm_bwd_post_kernel") or with_w:
        scalar_access("dn", "dn", 0, BH * N - 1)
    if kernel == "norm_chunk_sums_kernel" or (kernel in ("norm_fwd_kernel", "norm_bwd_post_kernel") and n_chunks > 1):
        scalar_access("ksum", "ksum", 0, BH * n_chunks * DP - 1)
        if with_w or kernel == "norm_bwd_post_kernel":
            scalar_access("wsum", "wsum", 0, BH * n_chunks * DP - 1)
    if kernel == "norm_bwd_post_kernel":
        assert l.grid[2] == (1 if p["only_dk"] else 2)
    # LDS: static arrays of NSEG * DP floats (twice with the weighted sums)
    assert (2 if with_w else 1) * NSEG * DP * 4 <= DEFAULT_LDS_LIMIT
    stats.workgroups += n_chunks * BH


# ---------------------------------------------------------------------------------------------
# plan-level checks of the walk kernels and the 256-row chunk kernels

def model_walk(arena: Arena, l: Launch, p: Dict, D: int, stats: Stats) -> None:
    rows = 128 if D <= 64 else 64
    N, BH, H = p["N"], p["BH"], p["H"]
    n_chunks, seg_chunks, n_seg = p["n_chunks"], p["seg_chunks"], p["n_seg"]
    assert n_chunks == -(-N // rows)
    assert seg_chunks >= 1 and n_seg >= 1 and (n_seg - 1) * seg_chunks < n_chunks <= n_seg * seg_chunks, \
        f"{l.kernel}: {n_seg} segments of {seg_chunks} chunks do not tile {n_chunks} chunks"
    assert l.grid[0] == 8 * ((BH + 7) // 8) * n_seg
    resident = 256 if D > 64 else 512
    assert BH * n_seg <= max(resident, BH), f"{l.kernel}: {BH * n_seg} workgroups for {resident} resident"
    for nm, ptr, sb, sh, sn, w in (("q", "q", "qs_b", "qs_h", "qs_n", p["wqk"]), ("k", "k", "ks_b", "ks_h", "ks_n", p["wqk"]),
                                   ("v", "v", "vs_b", "vs_h", "vs_n", p["wv"]), ("go", "go", "gs_b", "gs_h", "gs_n", p["wv"]),
                                   ("o", "o", "os_b", "os_h", "os_n", p["wv"]), ("dq", "dq", "dqs_b", "dqs_h", "dqs_n", p["wqk"]),
                                   ("dk", "dk", "dks_b", "dks_h", "dks_n", p["wqk"]), ("dv", "dv", "dvs_b", "dvs_h", "dvs_n", p["wv"])):
        if p[ptr]:
            lo, hi = tensor_extent(p, ptr, sb, sh, sn, H, BH, N, w)
            arena.require(f"{l.kernel} {nm}", lo, hi)
            assert p[ptr] % 16 == 0 and w % 8 == 0 and p[sn] % 8 == 0
            assert N * p[sn] * 2 <= 0x3fffffff
    E = D * D * 4
    if p["init"]:
        arena.require("entry states", p["init"], p["init"] + BH * n_seg * E)
    else:
        assert n_seg == 1 or l.kernel == "walk_bwd_kernel" and False, f"{l.kernel}: {n_seg} segments without entry states"
    if p["init_is_totals"]:  # (the walk adds up the segments' totals itself; a forward walk writes what it formed)
        assert D == 128 and n_seg >= 3 and p["init"], f"{l.kernel}: segment totals in place of entry states"
    if p["entry_out"]:
        assert p["init_is_totals"] and l.kernel in ("walk_fwd_kernel", "walk_fwd_wide_kernel")
        arena.require("entry states written by the walk", p["entry_out"], p["entry_out"] + BH * n_seg * E)
        assert not (p["init"] <= p["entry_out"] < p["init"] + BH * n_seg * E), "entry states over the totals"
    if p["xinit"]:
        arena.require("forward's entry states", p["xinit"], p["xinit"] + BH * n_seg * E)
    if p["xtotal"]:
        arena.require("forward's final states", p["xtotal"], p["xtotal"] + BH * E)
    if p["total_out"]:
        arena.require("final states", p["total_out"], p["total_out"] + BH * E)
    if p["saved"]:
        arena.require("per-chunk states", p["saved"], p["saved"] + BH * n_chunks * D * D * 2)
    for nm in ("zc", "rc"):
        if p[nm]:
            arena.require(nm, p[nm], p[nm] + BH * n_chunks * D * 4)
    for nm in ("denom", "dn"):
        if p[nm]:
            arena.require(nm, p[nm], p[nm] + BH * N * 4)
    stats.workgroups += BH * n_seg


def model_walk_wide(arena: Arena, l: Launch, p: Dict, stats: Stats) -> None:
    """One walk over both 128-column halves of a q / k of 129 .. 256 columns: the plan of a D = 128 walk
    whose q, k (dq, dk) rows are 128 + wqk2 wide, with a second set of states for the second half."""
    D, E = 128, 128 * 128 * 4
    assert p["wqk"] == 128 and 1 <= p["wqk2"] <= 128 and p["wqk2"] % 8 == 0 and not p["accumulate"]
    assert not p["init_transposed"] and not p["fmap"] and not p["denom"] and not p["dn"] and not p["saved"]
    if p["init_is_totals"]:  # (the walk adds up the segments' totals itself; what it forms goes to entry_out)
        assert 3 <= p["n_seg"] <= 7 and p["init"]
        if p["entry_out"]:
            assert l.kernel == "walk_fwd_wide_kernel"
            arena.require("entry_out", p["entry_out"], p["entry_out"] + p["BH"] * p["n_seg"] * E)
            assert not (p["init"] <= p["entry_out"] < p["init"] + p["BH"] * p["n_seg"] * E), "entry states over the totals"
    else:
        assert not p["entry_out"]
    whole = dict(p)
    whole["wqk"] = 128 + p["wqk2"]
    model_walk(arena, l, whole, D, stats)
    BH, n_seg = p["BH"], p["n_seg"]
    tiles = 6 if l.kernel == "walk_fwd_wide_kernel" else 8
    assert l.lds == tiles * 64 * 256 + 128 * 256, f"{l.kernel}: {l.lds} bytes of LDS"
    for first, second, count in (("init", "init2", BH * n_seg), ("xinit", "xinit2", BH * n_seg),
                                 ("total_out", "total_out2", BH), ("xtotal", "xtotal2", BH),
                                 ("entry_out", "entry_out2", BH * n_seg)):
        assert bool(p[first]) == bool(p[second]), f"{l.kernel}: {first} without {second} or the reverse"
        if p[second]:
            arena.require(f"{second} (second half)", p[second], p[second] + count * E)
            assert not (p[first] <= p[second] < p[first] + count * E) and \
                not (p[second] <= p[first] < p[second] + count * E), f"{l.kernel}: {first} and {second} overlap"


def model_walk_totals(arena: Arena, l: Launch, p: Dict, D: int, stats: Stats, both: bool = False) -> None:
    rows = 128 if D <= 64 else 64
    N, BH, H = p["N"], p["BH"], p["H"]
    n_chunks, seg_chunks, n_seg = p["n_chunks"], p["seg_chunks"], p["n_seg"]
    assert n_chunks == -(-N // rows) and (n_seg - 1) * seg_chunks < n_chunks <= n_seg * seg_chunks
    assert 0 <= p["seg_lo"] <= p["seg_hi"] <= n_seg
    assert l.grid[0] == 8 * ((BH + 7) // 8) * n_seg
    operands = [("y", "y", "ys_b", "ys_h", "ys_n", p["dy"]), ("z", "z", "zs_b", "zs_h", "zs_n", p["dz"])]
    if p["y2"]:  # a second Y operand (the other half of a wide q / k) in the same launch
        # (grid y picks the operand, or -- the kernel built for it -- every workgroup takes both: three sets of three tiles)
        assert l.grid[1] == (1 if both else 2) and not p["map_y"] and p["totals2"]
        assert not both or (D == 128 and p["dz"] <= 64 and l.lds == 9 * 64 * 256)
        operands.append(("y2", "y2", "ys_b", "ys_h", "ys_n", p["dy2"]))
        arena.require("segment totals of the second operand", p["totals2"], p["totals2"] + BH * n_seg * D * D * 4)
        assert not (p["totals"] <= p["totals2"] < p["totals"] + BH * n_seg * D * D * 4), "the two operands' totals overlap"
    else:
        assert l.grid[1] == 1 and not both
    for nm, ptr, sb, sh, sn, w in operands:
        lo, hi = tensor_extent(p, ptr, sb, sh, sn, H, BH, N, w)
        arena.require(f"totals {nm}", lo, hi)
    arena.require("segment totals", p["totals"], p["totals"] + BH * n_seg * D * D * 4)
    stats.workgroups += BH * n_seg


def check_all(arena: Arena, launches: List[Launch], stats: Stats) -> None:
    """Every launch of a call: the general limits, then the kernel's model."""
    for l in launches:
        stats.launches += 1
        stats.kernels[l.kernel] = stats.kernels.get(l.kernel, 0) + 1
        check_launch_limits(l)
        k, t = l.kernel, l.targs
        if k == "tri_xyt_z_fast_kernel":
            T, DC, DO, chunked, flags = t
            cfg = FastCfg(DC, DO, chunked)
            lds = cfg.SMEM + (cfg.STATE_BYTES if cfg.state_in_lds else 0)
            p = l.struct("a0")
            if chunked:
                assert p["state"], "chunk-wise kernel without a state"
                n_tiles = -(-p["N"] // cfg.BM)
                arena.require("chunk states", p["state"], p["state"] + p["BH"] * n_tiles * DC * DO * 2)
            model_tri_fast(arena, l, p, T, DC, DO, chunked, flags, lds, stats)
        elif k == "tri_xyt_z_fast_batch_kernel":
            T, DC, DO = t
            cfg = FastCfg(DC, DO, False)
            assert 1 <= l.grid[1] <= 3
            for i in range(l.grid[1]):
                model_tri_fast(arena, l, l.struct(f"a0.p{i}"), T, DC, DO, False, 0, cfg.SMEM, stats)
        elif k == "tri_xyt_z_fast_chunked_batch_kernel":
            T, DC, DO = t
            cfg = FastCfg(DC, DO, True)
            lds = cfg.SMEM + (cfg.STATE_BYTES if cfg.state_in_lds else 0)
            count = l.args["a1"]
            for i in range(count):
                p = l.struct(f"a0.p{i}")
                n_tiles = -(-p["N"] // cfg.BM)
                arena.require("chunk states", p["state"], p["state"] + p["BH"] * n_tiles * DC * DO * 2)
                model_tri_fast(arena, l, p, T, DC, DO, True, 0, lds, stats)
        elif k == "tri_pair_upper_kernel":
            model_tri_pair(arena, l, l.struct("a0"), t[1], stats)
        elif k == "tri_xyt_z_kernel":
            T, DC, DO = t
            model_tri_generic(arena, l, l.struct("a0"), DC, DO, stats)
        elif k.startswith("norm_") and k != "norm_scan_kernel":
            T, LPR, vec = t[0], t[1], t[2]
            with_w = bool(t[3]) if k == "norm_chunk_sums_kernel" else False
            model_norm(arena, l, l.struct("a0"), k, LPR, vec, with_w, stats)
        elif k == "norm_scan_kernel":
            ksum, wsum, BH, chunks, DP = (l.args[f"a{i}"] for i in range(5))
            assert l.grid[0] == -(-(BH * DP) // 256)
            arena.require("ksum", ksum, ksum + BH * chunks * DP * 4)
            if wsum:
                arena.require("wsum", wsum, wsum + BH * chunks * DP * 4)
        elif k in ("walk_fwd_kernel", "walk_bwd_kernel", "walk_dkdv_kernel", "walk_bwd_rev_kernel"):
            model_walk(arena, l, l.struct("a0"), t[1], stats)
        elif k in ("walk_fwd_wide_kernel", "walk_bwd_rev_wide_kernel"):
            model_walk_wide(arena, l, l.struct("a0"), stats)
        elif k == "walk_scan_kernel":
            totals, entry, n_seg, E, total2 = (l.args[f"a{i}"] for i in range(5))
            totals_b, entry_b = l.args["a8"], l.args["a9"]
            BH = total2 // (E // l.args["a6"] * (l.args["a7"] // 2))
            assert l.grid[1] == (2 if totals_b else 1) and bool(totals_b) == bool(entry_b)
            for t_, e_ in ((totals, entry),) + (((totals_b, entry_b),) if totals_b else ()):
                arena.require("segment totals", t_, t_ + BH * n_seg * E * 4)
                arena.require("entry states", e_, e_ + BH * n_seg * E * 4)
        elif k == "walk_totals_kernel":
            model_walk_totals(arena, l, l.struct("a0"), t[1], stats, both=len(t) > 4 and bool(t[4]))
        else:
            # remaining kernels (scans, vector sums, element-wise passes, chunk states): limits above,
            # and every pointer argument inside a tensor or the workspace
            for name, v in l.args.items():
                if isinstance(v, int) and v >= (1 << 40):
                    assert arena.find(v) is not None, f"{k}: argument {name} = {v:#x} points nowhere"
