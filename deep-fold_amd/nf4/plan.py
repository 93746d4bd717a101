"""Host-side mirror of the ``chr_nf4_gemm`` launch planner.

Pure Python, no GPU and no library: the same arithmetic as ``plan_impl`` in
``csrc/nf4_gemm.hip``, so grid sizes and workspace needs can be asserted
anywhere.  If the two diverge the library is the truth; ``tests/test_abi.py``
checks they agree.  Plays the part of the reference's ``gpu/nf4/plan.py:161-236``
for this library's gfx950 tiles.

Kernel families by token count ``N`` (the reference's name for it; out features
are ``M``, in features ``K``):

* ``N == 1``  row-streaming GEMV, no split-K (path ``GEMV``).
* ``N = 2..16`` / ``17..32``  MFMA tile, 128 rows per workgroup, split-K over ``grid_y``
  in slices of one to four K tiles, the length that costs the busiest compute unit least
  (``_pick_split_rows``; paths ``PREFILL`` / ``PREFILL_N32``).
* ``N = 33..64``  the same with twice the token columns, about three K tiles per workgroup
  and no more splits than reach 1.6 workgroups per compute unit
  (``PREFILL_N64``); launched only through ``chr_nf4_gemm_ws_max`` with ``max_n`` > 32,
  the plain entries keep the reference's ceiling of 32.

Two kernels serve the MFMA paths.  Slices of at most four K tiles (two above 32 columns) run
the row-streaming tile: 512 threads, every weight byte loaded straight into the register
that feeds the matrix core.  Longer slices (unsplit launches of a long K) run the K-tiled
one: 256 threads, weights staged through LDS one tile ahead.
"""

from __future__ import annotations

import os

from dataclasses import dataclass

__all__ = [
    "GEMV",
    "PREFILL",
    "PREFILL_N32",
    "PREFILL_N64",
    "ONE_WAVE",
    "GROUP_SIZE",
    "LIVE_MAX_N",
    "PLAN_MAX_N",
    "Plan",
    "k_pad",
    "gemv_rows_per_wavefront",
    "gemv_is_staged",
    "staged_lds_bytes",
    "gemm_streams",
    "gemm_streams_rows",
    "STAGED_MIN_CODES",
    "plan",
]

GEMV = 1
PREFILL = 2
PREFILL_N32 = 3
PREFILL_N64 = 4

GROUP_SIZE = 64

#: compute units of an MI355X; the unit the split-K target is expressed in when
#: the caller gives no ``one_wave`` and no device is visible.
ONE_WAVE = 256

#: live ``chr_nf4_gemm`` ceiling (``gpu/nf4/plan.py:57``)
LIVE_MAX_N = 32
#: the planner also describes N = 33..64 (``gpu/nf4/plan.py:59``)
PLAN_MAX_N = 64

_BM = 128
_BK = 256
_BLOCK = 256
_MAX_AUTO_SPLIT = 32
_TILES_PER_SPLIT = 3


def _gemm_lds(col_blocks: int) -> int:
    """codebook, staged activation tile (bf16, padded rows, ``col_blocks`` x 32 columns), and
    per wavefront (4) a weight area (32 rows of BK/2 + 16 bytes) and the tile's group scales"""
    return (64 + col_blocks * 32 * (_BK + 8) * 2 + 4 * 32 * (_BK // 2 + 16)
            + 4 * 32 * (_BK // 64) * 2)


_PATH_NAME = {GEMV: "gemv", PREFILL: "prefill", PREFILL_N32: "prefill_n32",
              PREFILL_N64: "prefill_n64"}


def k_pad(k: int) -> int:
    """``64 * ceil(K / 64)``."""
    return GROUP_SIZE * ((int(k) + GROUP_SIZE - 1) // GROUP_SIZE)


def _ceil_div(a: int, b: int) -> int:
    return -(-int(a) // int(b))


#: The staged GEMV kernel (x and a 64 KB level-pair table in LDS, 1024-thread workgroups, one
#: per compute unit) is taken from this many codes up, and whenever K is ragged.
STAGED_MIN_CODES = 16 << 20
_STAGED_TABLE_BYTES = 256 * 64 * 4
_STAGED_SMALL_BYTES = 512
_MAX_DYN_LDS = 150 * 1024


def staged_lds_bytes(k_pad_: int) -> int:
    """LDS of a staged GEMV launch: table, reduction scratch, x in half steps of 1024 codes and
    one float per lane and half step (the powers of two of the binary16 form)."""
    half_steps = _ceil_div(int(k_pad_) // 16, 64)
    return _STAGED_TABLE_BYTES + _STAGED_SMALL_BYTES + half_steps * 128 * 16 + half_steps * 64 * 4


def ring_piece_steps(half_steps: int) -> int:
    """Half steps per piece of the ring GEMV kernel for a row of ``half_steps``: the largest
    divisor in 4..7 (eight slots keep more bytes in flight than pays); for rows longer than a
    piece also the first of 7, 6, 5, 8 that divides ``half_steps + 1`` (the last piece then ends
    in one empty slot); 0 when that kernel does not take the row.  Gate/up pairs go through the
    same ring, one row after the other."""
    for ns in range(7, 3, -1):
        if half_steps % ns == 0:
            return ns
    if half_steps > 8:
        for ns in (7, 6, 5, 8):
            if (half_steps + 1) % ns == 0:
                return ns
    return 0


def ring_wanted() -> bool:
    """Whether staged launches go to the ring kernels where those take the row length: yes,
    unless ``CHR_NF4_GEMV_RING=0``."""
    return os.environ.get("CHR_NF4_GEMV_RING") != "0"


def gemv_is_staged(m: int, k: int, k_pad_: int | None = None) -> bool:
    """Kernel family ``chr_nf4_gemv`` takes for a plain launch (no fused norm)."""
    kp = k_pad(k) if k_pad_ is None else int(k_pad_)
    fits = staged_lds_bytes(kp) <= _MAX_DYN_LDS
    if int(k) != kp:
        return fits
    return fits and int(m) * kp >= STAGED_MIN_CODES


def gemv_rows_per_wavefront(m: int, forced: int = 0, staged: bool = False,
                            k_pad_: int | None = None) -> int:
    """Rows one wavefront of the GEMV walks together (they share x)."""
    if forced in (1, 2, 4):
        return forced
    if staged:
        if k_pad_ is not None and ring_wanted() and ring_piece_steps(_ceil_div(k_pad_ // 16, 64)):
            return 1
        return 2 if m >= 32768 else 1
    if m >= 32768:
        return 4
    return 2 if m >= 4096 else 1


@dataclass(frozen=True)
class Plan:
    path: int
    grid_x: int
    grid_y: int
    block: int
    bm: int
    bk: int
    n_ktiles: int
    tiles_per_split: int
    ctas: int
    smem_bytes: int
    ws_floats: int

    @property
    def path_name(self) -> str:
        return _PATH_NAME[self.path]

    @property
    def live(self) -> bool:
        """Launched by the entries that keep the reference's ceiling of 32 columns."""
        return self.path != PREFILL_N64


def gemm_streams_rows(N: int, tiles_per_split: int) -> bool:  # noqa: N803
    """Whether a launch runs the row-streaming tile (weights straight from global memory into
    the MFMA operand, the whole K slice requested at once) instead of the K-tiled one: slices
    of at most four K tiles, two for chunks wider than 32 columns.  ``CHR_NF4_GEMM_ROWS=0`` in
    the environment keeps the library on the K-tiled kernel; like the library, this mirror
    reads the switch once, when it is first needed."""
    return _rows_kernel_on() and tiles_per_split <= (2 if N > 32 else 4)


_ROWS_ON: bool | None = None


def _rows_kernel_on() -> bool:
    global _ROWS_ON
    if _ROWS_ON is None:
        raw = os.environ.get("CHR_NF4_GEMM_ROWS", "")
        try:
            _ROWS_ON = int(raw) != 0 if raw.strip() else True
        except ValueError:
            _ROWS_ON = False     # atoi() of a non-number is 0
    return _ROWS_ON


_STREAM_ON: int | None = None
_STREAM_ONLY: int | None = None
_STREAM_ROWS = 32
_STREAM_MAX_GROUPS = 96


def stream_lds_bytes(row_blocks: int) -> int:
    """LDS of the stream tile with ``row_blocks`` (1 or 2) 32-row blocks a workgroup: the pair
    table (32 copies of 256 entries), two chunks of x (32 token rows of 512 + 8), two chunks
    of weights (rows of 256 + 16 bytes), the rows' scales."""
    rows = _STREAM_ROWS * row_blocks
    return 256 * 32 * 4 + 2 * 32 * 520 * 2 + 2 * rows * 272 + _STREAM_MAX_GROUPS * rows * 2


#: LDS of the 64-column form: the pair table, two chunks of x (64 token rows of 256 + 8), two
#: chunks of weights (64 rows of 128 + 16 bytes), the scales of 64 rows and 80 groups
_STREAM_LDS_64 = 256 * 32 * 4 + 2 * 64 * 264 * 2 + 2 * 64 * 144 + 80 * 64 * 2


def _env_int_once(name: str, dflt: int) -> int:
    raw = os.environ.get(name, "")
    try:
        return int(raw) if raw.strip() else dflt
    except ValueError:
        return 0                 # atoi() of a non-number is 0


def stream_policy_default() -> int:
    """-1 never, 0 where the cost model prefers the stream tile, 1 wherever it fits: from
    ``CHR_NF4_GEMM_STREAM`` (0: never, 2: wherever it fits), read once like the library does
    (``nf4_gemm_stream_policy`` changes the library's; pass the same to ``plan``)."""
    global _STREAM_ON
    if _STREAM_ON is None:
        e = _env_int_once("CHR_NF4_GEMM_STREAM", 1)
        _STREAM_ON = -1 if e == 0 else (1 if e == 2 else 0)
    return _STREAM_ON


def _stream_columns(N: int, policy: int) -> bool:  # noqa: N803
    """Chunk widths the stream tile takes (8, 16, 24, 32, and 64 in a form of its own)."""
    return policy >= 0 and ((8 <= N <= 32 and N % 8 == 0) or N == 64)


_STREAM_SPLITS: bool | None = None
#: the stream tile's cost model, hundredths of a microsecond: a round of workgroups of 32 / 64
#: rows, a 512-wide chunk at 8 / 16 / 24 / 32 columns, the meeting of a split's partials
_STREAM_FIXED = (450, 600)
_STREAM_CHUNK = ((50, 52, 62, 73), (86, 93, 100, 106))
_STREAM_CHUNK_64 = 110      # a 256-wide chunk of the 64-column form (64 rows a workgroup)
_STREAM_MEET = 230
_STREAM_MAX_SPLIT = 8
_STREAM_MIN_CODES = 1 << 24
_STREAM_MIN_CODES_64 = 1 << 20    # at 64 columns the split tiles are slower
_ARRIVE_BLOCKS = 1024


def gemm_streams(M, N: int, k_pad_: int, force_split: int = 0,  # noqa: N803
                 one_wave: int = ONE_WAVE, have_ws: bool = True,
                 policy: int | None = None) -> tuple[int, int, int]:
    """``(row_blocks, split, chunks)`` of the stream tile for a launch, ``row_blocks`` 0 when
    another tile serves it.  The tile is a workgroup of sixteen wavefronts on 32 or 64 rows
    (``row_blocks`` 1 or 2) and ``chunks`` 512-wide chunks of K; ``split`` workgroups share a
    row block's K and the last of them to finish adds up their fp32 partials (no reduce
    launch); pair-table lookups, the scale applied per 64-wide group.  It takes whole-vector
    chunks of up to 32 columns (and, with 64 rows and 256-wide chunks, at most 20 of them a
    workgroup, chunks of exactly 64), no forced split, ``K_pad`` a multiple of 256, at most 12
    chunks a workgroup, splits only with a workspace and at most 8 of them, at most four rounds
    of workgroups (more than one only with 3072 of K or more a workgroup and the rounds four
    fifths full, and with splits only from 24 columns on) --
    and of the forms that fit, the cheapest by the cost model above (a split has to win by
    3%), if the launch has more than 2^24 weights, or 2^20 at 64 columns (``policy`` 0; 1: wherever it fits; -1:
    never; None: the process default).  ``M``: the rows, or the rows of each stacked matrix
    (blocks do not straddle matrices).  ``CHR_NF4_GEMM_STREAM_ROWS=32`` or ``64`` allows only
    that form and skips the weight count, ``CHR_NF4_GEMM_STREAM_SPLIT=0`` allows no splits.
    (The library also wants the scales 8-byte aligned, which device allocations are.)"""
    global _STREAM_ONLY, _STREAM_SPLITS
    if _STREAM_ONLY is None:
        _STREAM_ONLY = _env_int_once("CHR_NF4_GEMM_STREAM_ROWS", 0)
        _STREAM_SPLITS = _env_int_once("CHR_NF4_GEMM_STREAM_SPLIT", 1) != 0
    kp = int(k_pad_)
    rows = [int(M)] if isinstance(M, int) else [int(m) for m in M]
    best, best_cost = (0, 1, 0), 0
    policy = stream_policy_default() if policy is None else int(policy)
    if not (_stream_columns(N, policy) and force_split <= 0 and kp % _BK == 0):
        return best
    cus = int(one_wave)
    wide = N == 64              # 64 rows and chunks of 256 only, at most 20 a workgroup
    chunk_k, bodies = (256, 20) if wide else (512, 12)
    n_ch = _ceil_div(kp, chunk_k)
    for rb in ((2,) if wide else (1, 2)):
        if _STREAM_ONLY not in (0, _STREAM_ROWS * rb):
            continue
        blocks = sum(_ceil_div(m, _STREAM_ROWS * rb) for m in rows)
        for split in range(1, min(n_ch, _STREAM_MAX_SPLIT) + 1):
            chunks = _ceil_div(n_ch, split)
            if _ceil_div(n_ch, chunks) != split or chunks > bodies:
                continue
            rounds = _ceil_div(blocks * split, cus)
            if rounds > 4 or (split > 1 and (not _STREAM_SPLITS or not have_ws
                                             or blocks > _ARRIVE_BLOCKS)):
                continue
            if rounds > 1 and (chunks * chunk_k < 6 * 512 or blocks * split * 5 < rounds * cus * 4
                               or (split > 1 and N < 24)):
                continue
            per_chunk = _STREAM_CHUNK_64 if wide else _STREAM_CHUNK[rb - 1][N // 8 - 1]
            cost = rounds * (_STREAM_FIXED[rb - 1] + chunks * per_chunk)
            if split > 1:
                cost += _STREAM_MEET
                cost += cost // 32
            if best[0] == 0 or cost < best_cost:
                best, best_cost = (rb, split, chunks), cost
    if policy == 0 and _STREAM_ONLY == 0 and sum(rows) * kp <= (_STREAM_MIN_CODES_64 if wide
                                                                else _STREAM_MIN_CODES):
        return (0, 1, 0)
    if sum(rows) * kp >= 1 << 33:   # the tile addresses the packed bytes with 32-bit offsets
        return (0, 1, 0)
    return best


def _pick_split_rows(grid_x: int, n_ktiles: int, cus: int, fallback: int) -> int:
    """Split for the row-streaming tile (chunks of up to 32 columns): slices of 1..4 K tiles,
    cost = slices of the busiest compute unit x tiles (2 us each; 2.8 when a launch leaves one
    workgroup per unit) + 0.2 us per split, ties to the longer slice."""
    best, best_cost = 0, 0
    for tps in range(1, 5):
        split = _ceil_div(n_ktiles, tps)
        if split > _MAX_AUTO_SPLIT or _ceil_div(n_ktiles, split) != tps:
            continue
        rounds = _ceil_div(grid_x * split, cus)
        cost = rounds * tps * (28 if rounds == 1 else 20) + split * 2
        if best == 0 or cost <= best_cost:
            best, best_cost = split, cost
    return best if best > 0 else fallback


def _pick_split(grid_x: int, n_ktiles: int, N: int, have_ws: bool, force_split: int,  # noqa: N803
                one_wave: int) -> tuple[int, int]:
    want = 1
    if have_ws:
        # workgroups worth splitting for: 3 per compute unit, 1.6 for chunks wider than 32
        target = int(one_wave) * 8 // 5 if N > 32 else int(one_wave) * 3
        by_grid = max(1, _ceil_div(target, grid_x))
        by_tiles = _ceil_div(n_ktiles, _TILES_PER_SPLIT)
        want = force_split if force_split > 0 else min(_MAX_AUTO_SPLIT, by_tiles, by_grid)
        if force_split <= 0 and N <= 32:
            want = _pick_split_rows(grid_x, n_ktiles, int(one_wave), want)
    want = max(1, min(want, n_ktiles))
    tiles_per_split = _ceil_div(n_ktiles, want)
    return _ceil_div(n_ktiles, tiles_per_split), tiles_per_split


def plan(M: int, K: int, N: int = 1, *, K_pad: int | None = None, have_ws: bool = True,  # noqa: N803
         force_split: int = 0, one_wave: int = ONE_WAVE, gemv_rows: int = 0,
         stream_policy: int | None = None) -> Plan:
    M, K, N = int(M), int(K), int(N)
    if M < 1 or K < 1:
        raise ValueError(f"M and K must be >= 1, got M={M} K={K}")
    if not 1 <= N <= PLAN_MAX_N:
        raise ValueError(f"N={N} not in 1..{PLAN_MAX_N} (live launch is 1..{LIVE_MAX_N})")
    kp = k_pad(K) if K_pad is None else int(K_pad)
    if kp != k_pad(K):
        raise ValueError(f"K_pad={kp} != 64*ceil(K/64) = {k_pad(K)}")
    if N == 1:
        if gemv_is_staged(M, K, kp):
            # one workgroup of 16 wavefronts per compute unit; bm = rows it covers per pass
            bm = 16 * gemv_rows_per_wavefront(M, gemv_rows, staged=True, k_pad_=kp)
            n_ktiles = _ceil_div(kp, 1024)
            grid_x = min(int(one_wave), _ceil_div(M, bm))
            return Plan(GEMV, grid_x, 1, 1024, bm, 1024, n_ktiles, n_ktiles, grid_x,
                        staged_lds_bytes(kp), 0)
        bm = 4 * gemv_rows_per_wavefront(M, gemv_rows)
        n_ktiles = _ceil_div(kp, 2048)
        grid_x = _ceil_div(M, bm)
        lds = (16 + 16 + 16 * 4) * 4  # codebook + reduction partials + K-split partials
        return Plan(GEMV, grid_x, 1, 256, bm, 2048, n_ktiles, n_ktiles, grid_x, lds, 0)
    path = PREFILL if N <= 16 else (PREFILL_N32 if N <= 32 else PREFILL_N64)
    grid_x = _ceil_div(M, _BM)
    n_ktiles = _ceil_div(kp, _BK)
    row_blocks, split, chunks = gemm_streams(M, N, kp, force_split, one_wave, have_ws, stream_policy)
    if row_blocks:
        bm = _STREAM_ROWS * row_blocks
        grid_x = _ceil_div(M, bm)
        tps = chunks if N == 64 else min(2 * chunks, n_ktiles)
        lds = _STREAM_LDS_64 if N == 64 else stream_lds_bytes(row_blocks)
        return Plan(path, grid_x, split, 1024, bm, _BK, n_ktiles, tps, grid_x * split, lds,
                    split * M * N if split > 1 else 0)
    split, tps = _pick_split(grid_x, n_ktiles, N, have_ws, force_split, one_wave)
    ws = split * M * N if split > 1 else 0
    if gemm_streams_rows(N, tps):
        nc = 1 if N <= 16 else (2 if N <= 32 else 4)
        smem = 64 + nc * 16 * (tps * _BK + 8) * 2   # codebook + transposed activation slice
        return Plan(path, grid_x, split, 512, _BM, _BK, n_ktiles, tps, grid_x * split, smem, ws)
    smem = _gemm_lds(1 if N <= 32 else 2)
    return Plan(path, grid_x, split, _BLOCK, _BM, _BK, n_ktiles, tps, grid_x * split, smem, ws)
