"""Block-skip planner: which KV tiles a Q tile has to visit.

The reference derives these bounds at compile time with interval analysis over
the mask predicates plus z3/sympy (``loopfuse/compiler/passes/
skip_loop_iterations.py:267-378``): a KV-tile step whose every score is masked
leaves all carried variables unchanged and is cut off by tightening the loop's
``start``/``end``.  For the two masks the reference has (causal, causal sliding
window; ``loopfuse/torch_backend/ops.py:675-751``) the result has a closed
form, which is what the HIP prefill kernel evaluates per workgroup and what
this module states for the host (grid sizing, tests, flop accounting).

Contract (checked bit-exact against the dense mask in the tests):
    visited(qt) == { kt : any(mask[qt*BM:(qt+1)*BM, kt*BN:(kt+1)*BN]) }
"""
from __future__ import annotations

# (query rows per workgroup, KV rows per LDS tile) of each prefill kernel
TILE_SHAPES = {
    "prefill": (128, 64),        # lf_attn_prefill: 4 waves x 32 rows, two waves per SIMD
    "prefill_swp_pack": (32, 64),   # lf_attn_prefill_swp -DLF_GQAPACK=4: 32 rows x 4 query heads of one group
    "prefill_swp_pack2": (64, 64),  # lf_attn_prefill_swp -DLF_GQAPACK=2: 64 rows x 2 query heads of one group
    "prefill_swp": (128, 64),    # lf_attn_prefill_swp: 4 waves x 32 rows, direct-to-LDS staging, reads issued ahead
}
PREFILL_BM, PREFILL_BN = TILE_SHAPES["prefill"]


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def tile_range(mask: str | None, qt: int, Sq: int, Sk: int, window: int = 0,
               bm: int = PREFILL_BM, bn: int = PREFILL_BN) -> tuple[int, int]:
    """Half-open range [begin, end) of KV tiles visited by Q tile ``qt``.

    mask: None/"none", "causal" (j <= i) or "sliding" (j <= i and i - j < window);
    row i and column j are absolute positions, masks are top-left aligned.
    """
    nkt = cdiv(Sk, bn)
    q0 = qt * bm
    qlast = min(q0 + bm, Sq) - 1
    if qlast < q0:
        return (0, 0)
    begin, end = 0, nkt
    if mask in ("causal", "sliding"):
        # tile kt has a column j <= qlast  <=>  kt*bn <= qlast
        end = min(nkt, qlast // bn + 1)
    if mask == "sliding":
        if window < 1:
            raise ValueError("window must be >= 1")
        # the union over rows of [i-window+1, i] is [q0-window+1, qlast]; tile kt
        # reaches it iff its last column >= q0-window+1
        lo = q0 - window + 1
        if lo > 0:
            begin = lo // bn
    return (begin, max(begin, end))


def visited_tiles(mask: str | None, Sq: int, Sk: int, window: int = 0,
                  bm: int = PREFILL_BM, bn: int = PREFILL_BN) -> list[tuple[int, int]]:
    """tile_range for every Q tile."""
    return [tile_range(mask, qt, Sq, Sk, window, bm, bn) for qt in range(cdiv(Sq, bm))]


def executed_flops(mask: str | None, B: int, Hq: int, Sq: int, Sk: int, D: int, window: int = 0) -> int:
    """MFMA flops the prefill kernel issues (whole tiles), as opposed to the
    algorithmic count of the reference's benchmark (``tests/benchmark.py:110,
    280-284``)."""
    tiles = sum(e - b for b, e in visited_tiles(mask, Sq, Sk, window))
    return 4 * B * Hq * tiles * PREFILL_BM * PREFILL_BN * D
