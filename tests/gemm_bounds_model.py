"""Host-side replay of the address arithmetic of the int8 GEMM kernels (triton_int_amd/csrc/gemm_i8.hip).

For a problem (batch, M, N, K, strides, output type) and the launch the library plans for it
(ti_gemm_plan: configuration, K split, tile order, grid -- the same host code a real launch runs), this
module walks every workgroup of the grid, re-derives with numpy every global-memory access the kernel
makes (descriptor base and extent, per-lane vector offset, scalar offset, the software and hardware range
checks, in the kernels' own 32-bit arithmetic) and asserts that

  * every work item of a persistent kernel maps to a valid (batch, tile, split) and the items cover every
    output tile exactly once,
  * every descriptor extent and per-lane offset fits the 32-bit registers the kernel keeps them in,
  * every access that passes the range check lies inside its operand's allocation -- including the scalar
    offset, which the hardware adds AFTER the range check,
  * the set of output elements stored is exactly [0, M) x [0, N) of every batch entry, each once.

Operands are modelled as allocations of exactly the bytes the strides imply, so one byte out of range
fails.  No GPU and no kernel is involved; the model is a second, independent statement of the indexing,
and a disagreement between it and the kernel shows up in the GPU parity tests, not here.
"""
from __future__ import annotations

import ctypes
import re
from dataclasses import dataclass

import numpy as np

OOB = 0x80000000
ESZ = {0: 1, 1: 4, 2: 4, 3: 2, 4: 2}  # ti_dtype -> bytes


def _i32(x):
    """Wraps to signed 32 bits like the kernels' int arithmetic."""
    x = np.asarray(x, dtype=np.int64) & 0xFFFFFFFF
    return np.where(x >= 1 << 31, x - (1 << 32), x)


def _u32(x):
    return np.asarray(x, dtype=np.int64) & 0xFFFFFFFF


def _fits_i32(x, what):
    x = np.asarray(x, dtype=np.int64)
    assert x.size == 0 or (x.min() >= -(1 << 31) and x.max() < (1 << 31)), f"{what} overflows int32: {x.min()} .. {x.max()}"


@dataclass
class Problem:
    batch: int
    M: int
    N: int
    K: int
    sAb: int
    sAm: int
    sBb: int
    sBn: int
    sCb: int
    sCm: int
    out_dtype: int  # ti_dtype
    sAk: int = 1
    sBk: int = 1
    sCn: int = 1
    a_base: int = 1 << 20  # modelled device addresses (alignment is all that matters)
    b_base: int = 1 << 30
    c_base: int = 1 << 34

    @property
    def esz(self):
        return ESZ[self.out_dtype]

    def a_bytes(self):
        return (self.batch - 1) * self.sAb + (self.M - 1) * self.sAm + (self.K - 1) * self.sAk + 1 if self.K else 0

    def b_bytes(self):
        return (self.batch - 1) * self.sBb + (self.N - 1) * self.sBn + (self.K - 1) * self.sBk + 1 if self.K else 0

    def c_bytes(self):
        return ((self.batch - 1) * self.sCb + (self.M - 1) * self.sCm + (self.N - 1) * self.sCn + 1) * self.esz


def contiguous(batch, M, N, K, out_dtype) -> Problem:
    return Problem(batch, M, N, K, M * K, K, N * K, K, M * N, N, out_dtype)


@dataclass
class Plan:
    config: int
    splits: int
    kt_split: int
    tiles_m: int
    tiles_n: int
    group_m: int
    grid_x: int
    grid_y: int
    threads: int
    ksplit: int
    nwa: int
    partial_bytes: int
    name: str = ""


def plan_for(lib, pr: Problem, epilogue: int, bias_kind: int, config: int = -1, static_scratch: int = 0, round_mode: int = 0) -> Plan:
    """Asks the library (host code only, no GPU) what it would launch."""
    out = (ctypes.c_int64 * 12)()
    dummy = 1 << 12  # non-NULL, aligned, never dereferenced by a dry run
    rc = lib.ti_gemm_plan(pr.a_base, pr.sAb, pr.sAm, pr.sAk, pr.b_base, pr.sBb, pr.sBn, pr.sBk, pr.c_base, pr.sCb, pr.sCm, pr.sCn,
                          pr.batch, pr.M, pr.N, pr.K, dummy if bias_kind else None, bias_kind, dummy, dummy, epilogue,
                          pr.out_dtype, round_mode, config, static_scratch, out)
    assert rc == 0, f"ti_gemm_plan failed with {rc}: {lib.ti_last_error().decode()}"
    p = Plan(*[int(v) for v in out])
    p.name = lib.ti_gemm_config_name(p.config).decode()
    return p


# ---- tile order ---------------------------------------------------------------------------------

def tile_from_rank(pl: Plan, lid):
    lid = np.asarray(lid, dtype=np.int64)
    gsz = pl.group_m * pl.tiles_n
    gid = lid // gsz
    first_m = gid * pl.group_m
    gm = np.minimum(pl.tiles_m - first_m, pl.group_m)
    r = lid - gid * gsz
    return first_m + r % gm, r // gm


def persistent_items(pl: Plan, W: int):
    """Ranks of the work items every workgroup of a persistent launch walks: (workgroup, rank) arrays."""
    G = pl.grid_x
    wg, rank = [], []
    for b in range(G):
        if G & 7:
            first, step, count = b, G, ((W - b + G - 1) // G if b < W else 0)
        else:
            xcd, l, nb = b & 7, b >> 3, G >> 3
            per, rem = W >> 3, W & 7
            cnt = per + (1 if xcd < rem else 0)
            first = xcd * per + min(xcd, rem) + l
            step = nb
            count = (cnt - l + nb - 1) // nb if l < cnt else 0
        r = first + step * np.arange(count, dtype=np.int64)
        wg.append(np.full(count, b))
        rank.append(r)
    return np.concatenate(wg) if wg else np.zeros(0, np.int64), np.concatenate(rank) if rank else np.zeros(0, np.int64)


# ---- global -> LDS loads of the tiled kernels -------------------------------------------------

def _check_tile_loads(what, base_off, extent, rows0, ld, ROWS, BK, SWZ, K, k_lo, k_hi, alloc_bytes, chunk=256):
    """One operand tile per entry of base_off/extent/rows0 (arrays): lanes own chunks (row, clog); chunk clog
    of k-tile k is requested while k < K - 16*clog, else redirected out of range; the hardware drops a lane
    whose vector offset + 16 exceeds the descriptor's extent; the scalar offset k is added afterwards."""
    CH = BK // 16
    rows = np.arange(ROWS, dtype=np.int64)
    clog = np.arange(CH, dtype=np.int64)
    klim = K - clog * 16
    _fits_i32(extent, f"{what}: descriptor extent")
    assert (extent >= 0).all(), f"{what}: negative extent"
    for c0 in range(0, len(base_off), chunk):
        sl = slice(c0, c0 + chunk)
        voff = (rows0[sl, None, None] + rows[None, :, None]) * ld + clog[None, None, :] * 16  # [tile, row, chunk]
        _fits_i32(voff, f"{what}: vector offset")
        # the largest k (multiple of BK in [k_lo, k_hi)) at which the chunk is still requested
        k_last = np.minimum(k_hi[sl, None] - BK, ((klim[None, :] - 1) // BK) * BK)  # [tile, chunk]
        requested = k_last >= k_lo[sl, None]
        hw_ok = voff + 16 <= extent[sl, None, None]
        live = hw_ok & requested[:, None, :]
        addr_hi = base_off[sl, None, None] + voff + k_last[:, None, :] + 16
        addr_lo = base_off[sl, None, None] + voff + k_lo[sl, None, None]
        bad = live & ((addr_hi > alloc_bytes) | (addr_lo < 0))
        assert not bad.any(), f"{what}: {int(bad.sum())} lane loads leave the operand's {alloc_bytes} bytes (first at tile {c0 + np.argwhere(bad)[0][0]})"


# ---- stores of the persistent kernels' epilogue -------------------------------------------------

def _strip_bytes(wtn):
    s = wtn // 16
    return 32 * wtn if (s & (s - 1)) == 0 else 0


def _check_stream_stores(pr: Problem, bz, mw, nw, TM, TN, covered):
    """All stores of one consumer wave's (TM*32) x (TN*32) block at (mw, nw) of batch entry bz, replayed with
    the kernel's offset arithmetic (arrays over [instruction..., lane]); counts the stored elements in covered[bz]."""
    M, N, ldc, esz = pr.M, pr.N, pr.sCm, pr.esz
    c_extent = ((M - 1) * ldc + N) * esz
    _fits_i32(c_extent, "C extent")
    cbase = bz * pr.sCb * esz
    lane = np.arange(64, dtype=np.int64)
    lrow, lhi = lane & 31, lane >> 5
    WTN = TN * 32
    oob = _i32(OOB)

    def commit(voff, soff, nbytes, rows, cols, ncols):
        # hardware: a lane's store happens iff voff (unsigned) + nbytes <= extent; address = base + voff + soff
        voff, soff, rows, cols = np.broadcast_arrays(voff, soff, rows, cols)
        _fits_i32(soff, "scalar store offset")
        v = _u32(voff)
        ok = v + nbytes <= c_extent
        addr = cbase + v + soff
        bad = ok & ((addr < 0) | (addr + nbytes > pr.c_bytes()))
        assert not bad.any(), f"store outside C: batch {bz} block ({mw},{nw})"
        r, c = rows[ok], cols[ok]
        assert ((r >= 0) & (r < M)).all() and ((c >= 0) & (c + ncols <= N)).all(), f"store of an element outside M x N: batch {bz} block ({mw},{nw})"
        assert (addr[ok] == cbase + (r * ldc + c) * esz).all(), f"store address differs from the element's: batch {bz} block ({mw},{nw})"
        for k in range(ncols):
            np.add.at(covered[bz], (r, c + k), 1)

    if pr.out_dtype == 0:
        if _strip_bytes(WTN):
            SEG = WTN // 16
            RP = 64 // SEG
            r_row, r_seg = lane // SEG, lane % SEG
            s_rows_left = M - mw - r_row
            s_base = np.where(nw + r_seg * 16 < N, _i32((mw + r_row) * ldc + nw + r_seg * 16), oob)
            R = (np.arange(TM)[:, None] * 32 + np.arange(TN)[None, :] * RP).reshape(-1, 1)  # [store, 1]
            off = _i32(np.where(R < s_rows_left[None, :], s_base[None, :], oob) + _i32(R * ldc))
            commit(off, 0, 16, mw + R + r_row[None, :], nw + r_seg[None, :] * 16, 16)
        else:
            d_rows_left, d_cols_left = M - mw - lrow, N - nw - lhi * 16
            d_base = _i32((mw + lrow) * ldc + nw + lhi * 16)
            i = np.arange(TM).reshape(-1, 1, 1)
            j = np.arange(TN).reshape(1, -1, 1)
            inr = (i * 32 < d_rows_left) & (j * 32 < d_cols_left)
            off = _i32(np.where(inr, d_base, oob) + _i32(i * 32 * ldc + j * 32))
            commit(off, 0, 16, mw + i * 32 + lrow, nw + j * 32 + lhi * 16, 16)
        return
    pitch = ldc * esz
    rows_left = M - mw - 4 * lhi
    pairs = pr.out_dtype in (3, 4) and not (N & 1) and not (ldc & 1) and not (pr.sCb & 1) and not (pr.c_base & 3)
    i = np.arange(TM).reshape(-1, 1, 1, 1)
    if pairs:
        odd = lane & 1
        rows_left_pair = M - mw - odd
        r = np.arange(0, 16, 2).reshape(1, -1, 1, 1)
        h = np.arange(2).reshape(1, 1, -1, 1)
        for jp in range(TN // 2):
            n = nw + (2 * jp + lhi) * 32 + (lrow & ~1)
            base2 = np.where(n < N, _i32(((mw + odd) * ldc + n) * esz), oob)
            R = i * 32 + 8 * (r >> 2) + 4 * h + (r & 3)
            commit(np.where(R < rows_left_pair, base2, oob), R * pitch, 4, mw + R + odd, n, 2)
        if TN % 2 == 1:
            n = nw + (TN - 1) * 32 + (lrow & ~1)
            base = np.where(n < N, _i32(((mw + 4 * lhi + odd) * ldc + n) * esz), oob)
            R = (i * 32 + 8 * (r >> 2) + (r & 3))[:, :, 0]
            commit(np.where(R < rows_left - odd, base, oob), R * pitch, 4, mw + R + 4 * lhi + odd, n, 2)
        return
    r = np.arange(16).reshape(1, -1, 1, 1)
    R = (i * 32 + 8 * (r >> 2) + (r & 3))[:, :, 0]
    for j in range(TN):
        n = nw + j * 32 + lrow
        base = np.where(n < N, _i32(((mw + 4 * lhi) * ldc + n) * esz), oob)
        commit(np.where(R < rows_left, base, oob), R * pitch, esz, mw + R + 4 * lhi, n, 1)


# ---- the kernels --------------------------------------------------------------------------------

_TILED = re.compile(r"(ws|stream|mfma|shortk)_(\d+)x(\d+)x(\d+)_w(\d+)x(\d+)")


def check_launch(pr: Problem, pl: Plan, store_sample: int | None = 64, seed: int = 0) -> dict:
    """Replays the planned launch.  store_sample: the stores of at most that many consumer-wave blocks
    (the edge blocks always) are replayed element by element; None replays all (small problems).  Returns
    a few counts for reporting."""
    name = pl.name
    m = _TILED.match(name)
    rng = np.random.default_rng(seed)
    stats = {"config": name}
    if m:
        fam = m.group(1)
        BM, BN, BK, WM, WN = (int(m.group(i)) for i in range(2, 7))
        SWZ = int(re.search(r"_s(\d)", name).group(1)) if fam != "shortk" else 2
        assert pl.tiles_m == -(-pr.M // BM) and pl.tiles_n == -(-pr.N // BN)
        T = pl.tiles_m * pl.tiles_n
        KT = -(-pr.K // BK)
        persistent = fam != "mfma"
        if persistent:
            assert pl.grid_y == 1 and pl.threads <= 1024
            SPL = pl.splits
            W = T * pr.batch * SPL
            wg, rank = persistent_items(pl, W)
            assert np.array_equal(np.sort(rank), np.arange(W)), "the workgroups' items do not cover the work list exactly once"
            s = rank % SPL if SPL > 1 else np.zeros_like(rank)
            g = rank // SPL if SPL > 1 else rank
            bz, lid = g // T, g % T
            kt0 = s * pl.kt_split if SPL > 1 else np.zeros_like(rank)
            kts = np.minimum(pl.kt_split, KT - kt0) if SPL > 1 else np.full_like(rank, KT)
            assert (kts > 0).all() or KT == 0, "an empty K split"
            if SPL > 1:
                assert pr.batch == 1
                waves = WM * WN
                per_item = BM * BN * 4
                assert (rank.max() + 1) * per_item <= pl.partial_bytes, "split-K partial sums exceed the planned workspace"
                assert pl.partial_bytes <= 0x7FFFFFF0
                assert T * waves <= (1 << 16), "split-K ticket counters exceed the workspace's"
            if fam == "shortk":
                assert 16 <= pr.K <= 128 and KT <= 2
        else:
            assert pl.grid_x == T and pl.grid_y == pr.batch
            pid, by = np.meshgrid(np.arange(T, dtype=np.int64), np.arange(pr.batch, dtype=np.int64))
            pid, by = pid.ravel(), by.ravel()
            if pr.batch == 1:
                xcd, local = pid & 7, pid >> 3
                per, rem = T >> 3, T & 7
                lid = xcd * per + np.minimum(xcd, rem) + local
                bz = np.zeros_like(pid)
            else:
                Wt = T * pr.batch
                lin = by * T + pid
                xcd, local = lin & 7, lin >> 3
                per, rem = Wt >> 3, Wt & 7
                gg = xcd * per + np.minimum(xcd, rem) + local
                bz, lid = gg // T, gg % T
            assert np.array_equal(np.sort(bz * T + lid), np.arange(T * pr.batch)), "the grid does not cover every tile exactly once"
            kt0 = np.zeros_like(lid)
            kts = np.full_like(lid, KT)
        tm, tn = tile_from_rank(pl, lid)
        assert ((tm >= 0) & (tm < pl.tiles_m) & (tn >= 0) & (tn < pl.tiles_n) & (bz >= 0) & (bz < pr.batch)).all(), "a work item maps outside the tile grid"
        m0, n0 = tm * BM, tn * BN
        k_lo, k_hi = kt0 * BK, (kt0 + kts) * BK
        if KT > 0:
            if persistent:  # origin in the descriptor, offsets relative to the tile
                _check_tile_loads(f"{name} A", bz * pr.sAb + m0 * pr.sAm, _i32((pr.M - 1 - m0) * pr.sAm + pr.K), np.zeros_like(m0), pr.sAm, BM, BK, SWZ,
                                  pr.K, k_lo, k_hi, pr.a_bytes())
                _check_tile_loads(f"{name} B", bz * pr.sBb + n0 * pr.sBn, _i32((pr.N - 1 - n0) * pr.sBn + pr.K), np.zeros_like(n0), pr.sBn, BN, BK, SWZ,
                                  pr.K, k_lo, k_hi, pr.b_bytes())
            else:
                _check_tile_loads(f"{name} A", bz * pr.sAb, np.full_like(m0, _i32((pr.M - 1) * pr.sAm + pr.K)), m0, pr.sAm, BM, BK, SWZ, pr.K, k_lo, k_hi,
                                  pr.a_bytes())
                _check_tile_loads(f"{name} B", bz * pr.sBb, np.full_like(n0, _i32((pr.N - 1) * pr.sBn + pr.K)), n0, pr.sBn, BN, BK, SWZ, pr.K, k_lo, k_hi,
                                  pr.b_bytes())
        stats["items"] = int(len(lid))
        if persistent:
            # stores: once per output tile (the last split's item), one block per consumer wave
            WTM, WTN = BM // WM, BN // WN
            TMb, TNb = WTM // 32, WTN // 32
            tiles = np.unique(np.stack([bz, m0, n0], 1), axis=0)
            full = store_sample is None
            if not full:  # first and last batch entry only
                tiles = tiles[(tiles[:, 0] == 0) | (tiles[:, 0] == pr.batch - 1)]
            blocks = [(int(b), int(a) + wm * WTM, int(c) + wn * WTN) for b, a, c in tiles for wm in range(WM) for wn in range(WN)]
            if not full and len(blocks) > store_sample:
                edge = [x for x in blocks if x[1] + WTM > pr.M or x[2] + WTN > pr.N]
                inner = [x for x in blocks if not (x[1] + WTM > pr.M or x[2] + WTN > pr.N)]
                rng.shuffle(edge)
                rng.shuffle(inner)
                blocks = edge[:store_sample] + inner[:max(4, store_sample // 4)]
            else:
                full = True
            batches = {x[0] for x in blocks}
            covered = {b: np.zeros((pr.M, pr.N), np.int8) for b in batches}
            for b, mw, nw in blocks:
                _check_stream_stores(pr, b, mw, nw, TMb, TNb, covered)
            for b, cov in covered.items():
                if full:
                    assert (cov == 1).all(), f"batch {b}: {int((cov != 1).sum())} output elements not stored exactly once"
                else:
                    assert cov.max() <= 1, f"batch {b}: an output element stored twice"
            for b, mw, nw in blocks:
                sub = covered[b][max(mw, 0):min(mw + WTM, pr.M), max(nw, 0):min(nw + WTN, pr.N)]
                assert (sub == 1).all(), f"block ({mw},{nw}) of batch {b} not fully stored"
            stats["store_blocks"] = len(blocks)
        return stats
    if name.startswith("rows4"):
        NCH = -(-pr.K // 1024)
        NU = -(-pr.N // 4)
        assert pr.M <= 16 and pl.grid_y == pr.batch
        G = pl.grid_x
        per = -(-NU // G)
        NWA = pl.nwa
        KS = pl.ksplit if NWA == 8 else 1
        NSLOT = NWA // KS
        assert per <= NSLOT * 4 or KS == 1
        if NWA < 8:
            assert per <= NWA, "more units per workgroup than streaming waves"
        lane = np.arange(64, dtype=np.int64)
        kl = lane * 16
        units_seen = np.zeros(NU, np.int32)
        for b in range(G):
            ub0, ub1 = min(NU, b * per), min(NU, b * per + per)
            units_seen[ub0:ub1] += 1
        assert (units_seen == 1).all(), "the workgroups' weight-row units do not cover N exactly once"
        # weight loads: unit u rows 4u..4u+3 (clamped to N-1), chunk k0: requested while k0 + kl < K
        w_extent = _i32((pr.N - 1) * pr.sBn + pr.K)
        x_extent = _i32((pr.M - 1) * pr.sAm + pr.K)
        _fits_i32([(pr.N - 1) * pr.sBn + pr.K, (pr.M - 1) * pr.sAm + pr.K], "rows4 extents")
        k0 = np.arange(NCH, dtype=np.int64)[:, None] * 1024  # [chunk, lane]
        req = k0 + kl[None, :] < pr.K
        for rows, ld, extent, sb, alloc, what in ((np.minimum(np.arange(NU * 4), pr.N - 1), pr.sBn, w_extent, pr.sBb, pr.b_bytes(), "weights"),
                                                  (np.minimum(np.arange(16), pr.M - 1), pr.sAm, x_extent, pr.sAb, pr.a_bytes(), "activations")):
            voff = rows[:, None] * ld + kl[None, :]  # [row, lane]
            _fits_i32(voff, f"rows4 {what} offset")
            hw_ok = voff + 16 <= extent
            live = hw_ok[:, None, :] & req[None, :, :]
            addr = voff[:, None, :] + k0[None, :, :]
            for bzv in (0, pr.batch - 1):
                bad = live & (bzv * sb + addr + 16 > alloc)
                assert not bad.any(), f"rows4 {what}: load outside the operand"
        stats["units"] = NU
        return stats
    if name.startswith("skinny"):
        slab = int(re.search(r"slab(\d+)", name).group(1))
        MB = int(re.search(r"_m(\d+)", name).group(1)) // 16
        assert pr.M <= MB * 16
        ksplit = pl.ksplit
        groups = -(-pr.N // slab)
        assert pl.grid_x * (8 // ksplit) >= groups and pl.grid_y == pr.batch
        KSF = pr.K >> 6
        # raw pointer loads, 16 bytes per lane: lane (r16, c4) of a slab reads row min(row, last) at
        # c4*16 + 64*j for the whole k-steps j < KSF, and for the K tail at k0 = KSF*64 when its chunk is
        # inside K, else the first 16 bytes of its row
        c4 = np.arange(4, dtype=np.int64)
        for rows, ld, sb, alloc, what in ((np.minimum(np.arange(groups * slab), pr.N - 1), pr.sBn, pr.sBb, pr.b_bytes(), "weights"),
                                          (np.minimum(np.arange(MB * 16), pr.M - 1), pr.sAm, pr.sAb, pr.a_bytes(), "activations")):
            row_off = (pr.batch - 1) * sb + rows[:, None] * ld + c4[None, :] * 16
            if KSF:
                assert (row_off + (KSF - 1) * 64 + 16 <= alloc).all(), f"skinny {what}: k-step load outside the operand"
            if pr.K & 63:
                ok = KSF * 64 + c4 * 16 < pr.K
                tail = np.where(ok, KSF * 64, -c4 * 16)
                lo = row_off + tail[None, :]
                assert (lo >= 0).all() and (lo + 16 <= alloc).all(), f"skinny {what}: K-tail load outside the operand"
        return stats
    assert name.startswith("gather"), name
    return stats
