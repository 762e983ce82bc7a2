"""Tiling decisions for gfx950 (MI355X: 256 CUs in 8 XCDs, wave64, 512 VGPRs per lane, 160 KB LDS).

This is the analytic half of what the reference does by brute force (``QMatmulQFunc.lower``,
qfactory/core/qfunc.py:110-131, enumerates BLOCK_N x BLOCK_SIZE x NUM_ELM and times all of them):
given the problem it proposes one default tiling and a short list of neighbours worth timing.

Two regimes:

* ``gemv``  -- M small, HBM-bound.  Parameters of ``qf::GemvCfg`` (include/qf_gemv.hip.h):
  ``MT`` activation rows per block, ``WK`` waves along K per team, ``WN`` teams per block, ``U`` rows
  in flight per stage, ``STEPS`` stages per block, ``VB`` bytes per lane and load.
* ``mfma``  -- M large enough for the matrix cores.  Parameters of ``qf::MfmaCfg``
  (include/qf_mfma.hip.h): ``BM`` x ``BN`` block tile, ``WM`` x ``WNW`` wave grid, K-split ``KS``.
"""

NUM_CUS = 256
GEMV_MAX_M = 4          # largest M served by the dot2 GEMV before the MFMA kernel takes over
MFMA_AVAILABLE = False  # flipped once include/qf_mfma.hip.h provides qf::MfmaCfg / mfma_launch


def regime_for(M):
    return "gemv" if (M <= GEMV_MAX_M or not MFMA_AVAILABLE) else "mfma"


def elements_per_chunk(nbits, vb):
    return vb * 8 // nbits


def gemv_vec_bytes(K, nbits, group_size):
    """Widest per-lane load (16/8/4 bytes) that divides a packed row and stays inside one group."""
    row_bytes = K * nbits // 8
    for vb in (16, 8, 4):
        epc = elements_per_chunk(nbits, vb)
        if row_bytes % vb:
            continue
        if group_size is not None and group_size % epc:
            continue
        return vb
    raise ValueError(f"no vector width fits K={K}, nbits={nbits}, group_size={group_size}")


def _pow2_floor(x):
    p = 1
    while p * 2 <= x:
        p *= 2
    return p


def gemv_wave_split(K, nbits, vb, mt, max_waves=8, a_reg_budget=128):
    """(WK, IT) choices ranked by idle-lane waste, then by fewer waves."""
    epc = elements_per_chunk(nbits, vb)
    nch = K // epc
    a_regs_per_chunk = epc // 2
    out = []
    for wk in range(1, max_waves + 1):
        it = -(-nch // (64 * wk))
        if it * a_regs_per_chunk * mt > a_reg_budget:
            continue
        waste = (64 * wk * it - nch) / nch
        out.append((waste, wk * it, wk, it))
    if not out:
        wk = max_waves
        out.append((0.0, 0, wk, -(-nch // (64 * wk))))
    out.sort()
    return [(wk, it) for _, _, wk, it in out]


def gemv_tiling(M, N, K, nbits, group_size, wk=None, u=None, steps=None, wn=None, mt=None):
    """Default GEMV tiling; keyword arguments pin individual parameters."""
    vb = gemv_vec_bytes(K, nbits, group_size)
    if mt is None:
        mt = min(_pow2_floor(max(M, 1)), GEMV_MAX_M)
        if mt < M <= GEMV_MAX_M:
            mt *= 2                                   # 3 -> 4: one pass, one predicated row
    if wk is None:
        wk, it = gemv_wave_split(K, nbits, vb, mt)[0]
    else:
        it = -(-(K // elements_per_chunk(nbits, vb)) // (64 * wk))
    if u is None:
        # keep about 8 x 16 bytes of weight in flight per lane and stage, U*MT a power of two <= 64
        u = max(1, min(8 // it if it <= 8 else 1, 64 // mt))
        u = _pow2_floor(u)
    if wn is None:
        wn = max(1, 4 // wk)                          # blocks of about four waves
    if steps is None:
        # aim at >= 2 blocks per CU but let a team amortise its activation load over >= 8 rows
        rows_per_team = max(u, min(32, N // (2 * NUM_CUS * wn)))
        steps = max(1, rows_per_team // u)
    return {"MT": mt, "WK": wk, "WN": wn, "U": u, "STEPS": steps, "VB": vb}


def gemv_candidates(M, N, K, nbits, group_size):
    """Neighbourhood of the default worth timing on the device (deduplicated, default first)."""
    base = gemv_tiling(M, N, K, nbits, group_size)
    vb, mt = base["VB"], base["MT"]
    seen, out = set(), []

    def add(cfg):
        key = tuple(sorted(cfg.items()))
        if key not in seen and cfg["U"] * cfg["MT"] <= 64 and 64 * cfg["WK"] * cfg["WN"] <= 1024:
            seen.add(key)
            out.append(cfg)

    add(base)
    for wk, it in gemv_wave_split(K, nbits, vb, mt)[:3]:
        for u in (2, 4, 8):
            if u * it > 16:
                continue
            for wn in (1, 2, 4):
                if wk * wn > 8:
                    continue
                for steps in (1, 2, 4):
                    add({"MT": mt, "WK": wk, "WN": wn, "U": u, "STEPS": steps, "VB": vb})
    return out
