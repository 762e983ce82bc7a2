"""Tiling decisions for gfx950 (MI355X: 256 CUs in 8 XCDs, wave64, 512 VGPRs per lane, 160 KB LDS).

This is the analytic half of what the reference does by brute force (``QMatmulQFunc.lower``,
qfactory/core/qfunc.py:110-131, enumerates BLOCK_N x BLOCK_SIZE x NUM_ELM and times all of them):
given the problem it proposes one default tiling and a short list of neighbours worth timing.

Five kernel families (``regime_for`` picks one):

* ``gemv``  -- M < 3 (and 3-bit M <= 2), HBM-bound, v_dot2.  Parameters of ``qf::GemvCfg``
  (include/qf_gemv.hip.h): ``MT`` activation rows per block, ``WK`` waves along K per team, ``WN``
  teams per block, ``U`` rows in flight per stage, ``STEPS`` stages per block, ``VB`` bytes per lane
  and load.
* ``mgemv`` -- 3 <= M <= 32 when the activations fit the register file: persistent A-stationary MFMA
  kernel, ``qf::MGemvCfg`` (include/qf_mgemv.hip.h): ``MT16`` 16-row activation tiles, ``WK`` waves x
  ``CH`` chunks covering K, ``PB`` blocks, ``PF`` weight tiles in flight.  Long rows (K >= 7168, 3 <= M <= 16;
  narrow layers up to 32 rows): ``KS`` blocks split K and meet through scratch memory (``mgemv_ksplit_tiling``).
* ``skinny`` -- 3 <= M <= 16 where ``mgemv`` cannot hold the activations and K is not split over blocks
  (``ksplit=False``: layers with the norm prologue or the SwiGLU epilogue; what the split does not take):
  ``qf::SkinnyCfg`` (include/qf_skinny.hip.h): activations streamed per K-step instead of resident,
  ``WK`` waves splitting K, ``SB`` tiles per batch, ``D`` stages in flight, ``AST`` resident fragments.
* ``gemm``  -- larger M (and what ``mgemv`` cannot hold): ``qf::GemmCfg`` (include/qf_gemm.hip.h):
  ``BM`` activation rows per block, ``NT32`` 32-row weight tiles per wave, ``WN`` waves along N,
  ``WK`` wave groups along K, ``PA`` activation tiles in flight.
* ``mfma``  -- generic fallback, ``qf::MfmaCfg`` (include/qf_mfma.hip.h).
"""
import json
import os

NUM_CUS = 256
GEMV_MAX_M = 4          # largest M served by the dot2 GEMV before the MFMA kernel takes over
MFMA_AVAILABLE = True


MGEMV_MIN_M = 3         # below: dot2 GEMV; [MGEMV_MIN_M, MGEMV_MAX_M]: A-stationary MFMA kernel
MGEMV_MAX_M = 32


def regime_for(M, K=None, nbits=None, group_size=None, N=None, ksplit=True):
    if M < MGEMV_MIN_M or not MFMA_AVAILABLE:
        return "gemv"
    if ksplit and K is not None and mgemv_ksplit_tiling(M, N or 0, K, nbits, group_size) is not None:
        return "mgemv"
    if K is not None and nbits == 3:
        # 3-bit has three kernels: the dot2 GEMV (any M, tiled over grid.y), the A-stationary kernel and the GEMM
        if M <= MGEMV_MAX_M and mgemv_tiling(M, 0, K, nbits, group_size) is not None:
            return "mgemv"
        return "gemm" if gemm_supported(K, nbits, group_size) else "gemv"
    if K is None:
        return "gemv"
    if not mfma_supported(K, nbits, group_size):
        # K is not a whole number of 16-byte lane loads: only the GEMM (64-element iterations) and the dot2 GEMV remain
        return "gemm" if M > GEMV_MAX_M and gemm_supported(K, nbits, group_size) else "gemv"
    if M <= MGEMV_MAX_M and mgemv_tiling(M, 0, K, nbits, group_size) is not None:
        return "mgemv"
    if skinny_preferred(M, K, nbits, group_size, N):
        return "skinny"
    if M <= GEMV_MAX_M:
        return "gemv"
    # above 32 rows, or when the A-stationary kernel cannot hold the activations of this K in
    # registers: the LDS-staged GEMM (with a 32-row tile for small M)
    if gemm_supported(K, nbits, group_size):
        return "gemm"
    return "mfma"


def plane_bits(nbits):
    """Field width of the main weight plane: 3-bit rows are a 2-bit plane plus a 1-bit plane."""
    return 2 if nbits == 3 else nbits


def elements_per_chunk(nbits, vb):
    return vb * 8 // plane_bits(nbits)


def gemv_vec_bytes(K, nbits, group_size, mt=None, N=None):
    """Widest per-lane load (16/8/4 bytes of the main plane) that divides a packed row and stays
    inside one group; 3-bit rows need at least 8 (one whole word of the 1-bit plane per chunk).
    One activation row against a 2-bit main plane (2- and 3-bit weights, ``mt == 1``): 8 bytes -- 32 fields --
    per lane where the row then still fits one pass of eight waves.  Sixteen bytes are 64 fields and 32 activation
    registers per lane and half as many waves; measured at M = 1, cold weights, sixteen against eight bytes:
    2 bits 3.80 -> 3.02 us on 4096 x 4096, 8.86 -> 7.05 on 22016 x 4096, 6.10 -> 5.63 on 8192 x 8192, 29.6 -> 28.2 on
    57344 x 8192; 3 bits 4.93 -> 3.64, 12.9 -> 10.9, 8.55 -> 8.17, but 43.5 -> 48.4 on 57344 x 8192 (its 1-bit plane
    then comes in 4-byte loads), so 3-bit launches of many rounds of waves keep sixteen."""
    row_bytes = K * plane_bits(nbits) // 8
    widths = (16, 8) if nbits == 3 else (16, 8, 4)
    waves8 = -(-(K // elements_per_chunk(nbits, 8)) // 64)
    if mt == 1 and plane_bits(nbits) == 2 and waves8 <= 8:
        many_rounds = N is not None and (N * waves8) // 4 > 2 * 8 * 4 * NUM_CUS
        if not (nbits == 3 and many_rounds):
            widths = (8, 16) if nbits == 3 else (8, 16, 4)
    for vb in widths:
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
    """(WK, IT) choices ranked by idle-lane waste in steps of an eighth, then by fewer chunks per lane (more
    waves): up to ~12 % of idle lanes cost less than a third pass over the row (8192 x 29696: eight waves x
    two chunks, 10 % idle, 25.0 us against 34.4 us for five waves x three chunks, 3 % idle)."""
    epc = elements_per_chunk(nbits, vb)
    nch = K // epc
    a_regs_per_chunk = epc // 2
    out = []
    for wk in range(1, max_waves + 1):
        it = -(-nch // (64 * wk))
        if it * a_regs_per_chunk * mt > a_reg_budget:
            continue
        waste = (64 * wk * it - nch) / nch
        out.append((int(waste * 8), it, round(waste, 3), wk, it))
    if not out:
        wk = max_waves
        out.append((0, 0, 0.0, wk, -(-nch // (64 * wk))))
    out.sort()
    return [(wk, it) for _, _, _, wk, it in out]


_GEMV_TUNED = None


def gemv_tuned(M, N, K, nbits, group_size):
    """Winner of an on-device sweep over dot2 GEMV tilings for exactly this problem, or None
    (``gemv_tuned_gfx950.json`` beside this file, keyed like ``$QFACTORY_CONFIG``: "bits-M-N-K-group")."""
    global _GEMV_TUNED
    if _GEMV_TUNED is None:
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemv_tuned_gfx950.json")
        try:
            with open(path) as f:
                _GEMV_TUNED = json.load(f)
        except FileNotFoundError:
            _GEMV_TUNED = {}
    entry = _GEMV_TUNED.get(f"{nbits}-{M}-{N}-{K}-{group_size}")
    return dict(entry) if entry else None


def gemv_tiling(M, N, K, nbits, group_size, wk=None, u=None, steps=None, wn=None, mt=None):
    """Default GEMV tiling: the swept winner where one is stored for the exact problem, else the model below;
    keyword arguments pin individual parameters (and skip the table)."""
    if wk is None and u is None and steps is None and wn is None and mt is None:
        tuned = gemv_tuned(M, N, K, nbits, group_size)
        if tuned is not None:
            return tuned
    return gemv_tiling_model(M, N, K, nbits, group_size, wk, u, steps, wn, mt)


def gemv_tiling_model(M, N, K, nbits, group_size, wk=None, u=None, steps=None, wn=None, mt=None):
    """The analytic default alone."""
    if mt is None:
        mt = min(_pow2_floor(max(M, 1)), GEMV_MAX_M)
        if mt < M <= GEMV_MAX_M:
            mt *= 2                                   # 3 -> 4: one pass, one predicated row
    vb = gemv_vec_bytes(K, nbits, group_size, mt, N)
    if wk is None:
        # one activation row: up to sixteen waves per row when that makes one chunk per lane (8192 x 28672 at 4 bits:
        # fourteen waves x one chunk 21.8 us against seven x two 24.1, cold weights)
        wk, it = gemv_wave_split(K, nbits, vb, mt, max_waves=16 if mt == 1 else 8)[0]
    else:
        it = -(-(K // elements_per_chunk(nbits, vb)) // (64 * wk))
    # Loads in flight per lane (rows x chunks per row), measured on MI355X once the kernel's address
    # arithmetic had moved to scalar registers:
    #   * launches of at most ~2 rounds of resident waves (the 7B shapes): 4 loads, two teams per
    #     block, one stage -- many small waves (61 registers, 8 per SIMD) beat deeper stages;
    #   * larger launches (57344 x 8192: 7 rounds) or rows longer than one pass of the team
    #     (K = 28672): 8 loads, one team per block, and a second stage when a lane holds two chunks
    #     (46.6 -> 40.5 us and 37.6 -> 25.5 us);
    #   * 2- and 3-bit rows are short in bytes and heavy in decode work: 8 loads.
    big = it >= 2 or (N * wk) // 4 > 2 * 8 * 4 * NUM_CUS
    u_free, wn_free, steps_free = u is None, wn is None, steps is None
    if u is None:
        in_flight = 8 if (big or nbits <= 3) else 4
        if nbits == 3 and vb == 8 and mt == 1:
            in_flight = 4                             # two planes per row: four rows are eight loads (8192 x 8192: 7.94 us against 8.36)
        if nbits == 4 and it == 1 and wk == 4 and mt == 1:
            # K = 8192 at 4 bits (four waves per row): eight rows per stage with one scale / zero-point load per lane
            # and stage measured 8.26 us on 8192 x 8192 against 8.85 for four (cold weights)
            in_flight = 8
        u = max(1, min(in_flight // it if it <= in_flight else 1, 64 // mt, in_flight))
        u = _pow2_floor(u)
    if wn is None:
        wn = 1 if big else (2 if wk * 2 <= 12 else 1)         # 5120 x 13824, seven waves per team: one team 9.2 us, two 10.2
    if steps is None:
        steps = 2 if (big and it >= 2) else 1
        # several activation rows per block: 69 registers instead of 28 leave room for fewer resident
        # blocks, so the launch runs in two generations of short-lived blocks; four stages per block
        # spread the activation staging over more rows (M = 2: 13.9 -> 12.8 us on 22016 x 4096,
        # 11.2 -> 10.1 on 8192 x 8192) as long as every CU still gets a block
        if mt >= 2 and it == 1 and N // (wn * u * 4) >= NUM_CUS:
            steps = 4
    blocks16 = -(-N // 16)
    whole_rounds = blocks16 <= NUM_CUS or blocks16 % NUM_CUS == 0 or blocks16 >= 4 * NUM_CUS
    if mt == 1 and it == 1 and wk >= 6 and nbits == 4 and whole_rounds and u_free and wn_free and steps_free:
        # long rows, one chunk per lane: a team's activations are 22 KB and more, so four stages of four rows per
        # team and one team per block (cold weights: 4096 x 11008 5.97 us against 6.59 for two teams of one stage,
        # 3584 x 18944 8.30 against 9.48) -- where sixteen-row blocks fill the CUs evenly (5120 x 13824, 320 blocks:
        # 10.4 against 8.85 us for one stage)
        u, wn, steps = 4, 1, 4
    return {"MT": mt, "WK": wk, "WN": wn, "U": u, "STEPS": steps, "VB": vb}


def gemv_chunks_per_lane(K, nbits, cfg):
    """IT of qf::GemvCfg: chunks of VB bytes a lane owns per row."""
    nch = K // elements_per_chunk(nbits, cfg["VB"])
    return -(-nch // (64 * cfg["WK"]))


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


# --------------------------------------------------------------------------------------------
# MFMA regime
# --------------------------------------------------------------------------------------------

def mfma_supported(K, nbits, group_size):
    """The matrix-core kernel needs whole K-iterations and a lane's 16 bytes inside one group."""
    if nbits not in (2, 4, 8):
        return False
    epl = 128 // nbits
    return K % (4 * epl) == 0 and group_size % epl == 0


def mfma_tiling(M, N, K, nbits, group_size, **pins):
    """Default tile shape: AT x BT 16-row tiles per wave, WM x WN x WK waves per block."""
    m16 = -(-M // 16)
    if m16 <= 4:
        at, wm = m16, 1
    elif m16 <= 8:
        at, wm = (m16 + 1) // 2, 2
    else:
        at, wm = 4, 4
    bt = 2
    wn = max(1, 4 // wm)
    iters = K // (4 * (128 // nbits))
    wk = 1
    # small tiles leave the machine empty: split K over waves of the block until there are
    # 8 waves per block or the K-iterations run out
    while wm * wn * wk < 8 and wk * 2 <= iters and m16 <= 2:
        wk *= 2
    # too few blocks for 256 CUs: narrow the block along N
    while (N // (wn * bt * 16)) < 2 * NUM_CUS and wn > 1:
        wn //= 2
    if (N // (wn * bt * 16)) < NUM_CUS and bt > 1:
        bt = 1
    # the double-buffered activation tile (BM x 4*128/nbits elements) must fit LDS: fewer rows per block at 2 bits
    while mfma_lds_bytes(at, bt, wm, wn, wk, nbits) > 160 * 1024 and at > 1:
        at //= 2
    while mfma_lds_bytes(at, bt, wm, wn, wk, nbits) > 160 * 1024 and wm > 1:
        wm //= 2
    cfg = {"AT": at, "BT": bt, "WM": wm, "WN": wn, "WK": wk}
    cfg.update(pins)
    return cfg


def mfma_lds_bytes(at, bt, wm, wn, wk, nbits):
    """LDS of qf::mfma_kernel: two activation tiles per K-slice plus the partial tiles of a K split."""
    bk = 4 * (128 // nbits)
    return 2 * wk * (at * wm * 16) * (bk + 8) * 2 + ((wk - 1) * wm * wn * at * bt * 1024 if wk > 1 else 0)


def mfma_candidates(M, N, K, nbits, group_size):
    base = mfma_tiling(M, N, K, nbits, group_size)
    seen, out = set(), []
    iters = K // (4 * (128 // nbits))

    def add(cfg):
        key = tuple(sorted(cfg.items()))
        threads = 64 * cfg["WM"] * cfg["WN"] * cfg["WK"]
        if key in seen or threads > 1024 or cfg["WK"] > iters or cfg["AT"] * cfg["BT"] > 32:
            return
        if mfma_lds_bytes(cfg["AT"], cfg["BT"], cfg["WM"], cfg["WN"], cfg["WK"], nbits) > 160 * 1024:
            return
        seen.add(key)
        out.append(cfg)

    add(base)
    m16 = -(-M // 16)
    for wm in (1, 2, 4):
        at = -(-m16 // wm)
        if at > 8:
            at = 4
        for bt in (1, 2, 4):
            for wn in (1, 2, 4):
                for wk in (1, 2, 4):
                    add({"AT": at, "BT": bt, "WM": wm, "WN": wn, "WK": wk})
    return out


def mfma_cfg_string(problem, t, decode_strategy, nt_b):
    b = lambda x: "true" if x else "false"
    return (f"qf::MfmaCfg<{problem['NBITS']}, {problem['GS']}, {b(problem['SYM'])}, {problem['N']}, {problem['K']}, "
            f"{t['AT']}, {t['BT']}, {t['WM']}, {t['WN']}, {t['WK']}, {b(nt_b)}>")


# --------------------------------------------------------------------------------------------
# A-stationary MFMA regime (2 <= M <= 64)
# --------------------------------------------------------------------------------------------

def mgemv_supported(K, nbits, group_size):
    """Whole chunks of 16 bytes of the main plane per lane, and a lane's fields inside one group."""
    if nbits not in (2, 3, 4, 8) or not group_size or group_size <= 0:
        return False
    epl = 128 // plane_bits(nbits)
    return K % (4 * epl) == 0 and group_size % epl == 0


def mgemv_regs(mt16, ch, pf, nbits):
    """Rough VGPR need of qf::mgemv_kernel: resident activations, the ring of weight stages and
    the fragment copy of the tile being consumed (3-bit: plus the 1-bit plane of both)."""
    ksteps = (128 // plane_bits(nbits)) // 8
    hi = (pf * 4 * -(-ch // 2) + 2 * ch) if nbits == 3 else 0
    return mt16 * ch * ksteps * 4 + pf * (ch * 4 + 4) + ch * 4 + 48 + hi


def mgemv_lds_bytes(mt16, wk, ch, nbits, sb=4):
    """LDS of qf::mgemv_kernel: SB partial tiles per wave plus the wave's transposition buffer."""
    chunk = 4 * (128 // plane_bits(nbits))
    wbuf = max(16 * (ch * 64 + 16) + (16 * (ch * 32 + 16) if nbits == 3 else 0), 16 * (chunk * 2 + 16))
    return wk * sb * mt16 * 1024 + wk * wbuf


def mgemv_reg_limit(wk):
    waves_per_simd = -(-wk // 4)
    return min(512, 512 // waves_per_simd)


def mgemv_tiling(M, N, K, nbits, group_size, max_waves=16, **pins):
    """MT16 activation tiles resident per wave, WK waves x CH chunks covering K, PF weight tiles in
    flight; None if the activations do not fit the register file of one block."""
    if not mgemv_supported(K, nbits, group_size):
        return None
    chunk = 4 * (128 // plane_bits(nbits))
    if group_size % chunk and chunk % group_size:
        return None
    mt16 = -(-M // 16)
    nchunk = K // chunk
    best = None
    for ch in (16, 8, 4, 2, 1):
        if ch > nchunk:
            continue
        wk = -(-nchunk // ch)
        if wk > max_waves or (wk - 1) * ch >= nchunk:
            continue
        for pf in (1, 2, 4):
            if mgemv_regs(mt16, ch, pf, nbits) > mgemv_reg_limit(wk):
                continue
            if mgemv_lds_bytes(mt16, wk, ch, nbits) > 160 * 1024:
                continue
            waste = wk * ch - nchunk
            # more, thinner waves measured best on MI355X; with 8 - 16 waves per CU one tile ahead per
            # wave is enough (two ahead measured 3 - 8 % slower, four 5 - 150 % slower)
            key = (waste > ch // 2, -wk, pf != 1, waste)
            if best is None or key < best[0]:
                best = (key, wk, ch, pf)
    if best is None:
        return None
    _, wk, ch, pf = best
    cfg = {"MT16": mt16, "WK": wk, "CH": ch, "PB": NUM_CUS, "PF": pf}
    cfg.update(pins)
    return cfg


KSPLIT_MIN_K = 7168         # shortest rows the A-stationary kernel splits over several blocks
KSPLIT_NARROW_MIN_K = 5120          # ... on layers of KSPLIT_NARROW_N[0] .. [1] columns
KSPLIT_NARROW_N = (4096, 7168)
KSPLIT_MAX_M = 16
KSPLIT_WAVE_K = 256         # elements of K whose activations one wave keeps in registers
KSPLIT_BITS = (2, 3, 4, 8)


def mgemv_ksplit_tiling(M, N, K, nbits, group_size):
    """The A-stationary kernel with K split over KS blocks (``KS`` in the tiling; include/qf_mgemv.hip.h), for long rows
    and 3 .. 16 activation rows; None where it does not apply.

    A block then holds the activations of K / KS elements only -- sixteen waves of 256 elements each, the form that
    measured best at K = 4096 -- and the KS partial results meet through a scratch buffer in device memory.  Measured on
    MI355X (4 bits, groups of 128, cold weights, us per launch at M = 4 / 16, the kernel that served the shape before
    -> split): 8192 x 8192 14.4 / 14.6 -> 10.9 / 12.1; 16384 x 16384 57.4 / 78.0 -> 30.1 / 32.2; 4096 x 11008 10.4 /
    12.7 -> 9.4 / 10.3; 5120 x 13824 20.4 / 26.1 -> 14.7 / 15.5; 8192 x 28672 55.6 / 44.9 -> 28.2 / 29.8; 57344 x 8192
    53.8 / 57.3 -> 48.4 / 49.7; 4096 x 7168 8.2 / 9.4 -> 7.4 / 7.8.  Shorter rows lose (15360 x 5120 11.6 -> 13.2,
    22016 x 4096 12.1 -> 15.5: one block per CU already holds all of K there, and the split only adds the meeting), and
    so does M = 2 against the dot2 kernel (8192 x 8192 8.6 -> 10.5).  KS is the smallest power of two that leaves a
    block at most 4096 elements: more blocks than needed measured 15 - 30 % slower, fewer and fatter waves 3 - 50 %.
    8 bits, the streaming kernel -> split: 8192 x 8192 20.1 / 22.1 -> 16.7 / 18.1, 16384 x 16384 116 / 121 -> 52 / 53,
    4096 x 11008 13.7 / 17.2 -> 13.8 / 15.0.  2 and 3 bits: only where the unsplit kernel cannot hold the activations
    (4096 x 12288: 10.2 / 11.8 -> 10.1 / 10.4 at 2 bits, 23.2 / 23.5 -> 11.6 / 11.8 at 3; 16384 x 16384 at 2 bits 62 / 107
    -> 38 / 38); at K = 8192 the unsplit kernel is 1 - 2 us ahead."""
    if nbits not in KSPLIT_BITS or not (MGEMV_MIN_M <= M <= 2 * KSPLIT_MAX_M) or K < KSPLIT_NARROW_MIN_K:
        return None
    if K < KSPLIT_MIN_K and (nbits != 4 or M > KSPLIT_MAX_M or not N or not (KSPLIT_NARROW_N[0] <= N <= KSPLIT_NARROW_N[1])):
        # rows of 5120 .. 7167: two blocks along K pay on layers of about one tile per block only, now that the blocks'
        # sums meet in one trip to memory (us at M = 4 / 16, unsplit -> split: 5120 x 5120 8.2 / 8.5 -> 7.1 / 7.4, 7168 x 5120
        # 8.6 / 8.7 -> 7.9 / 8.3, 4096 x 6144 6.0 / 6.6 -> 5.8 / 6.3; 8192 x 5120 and 8192 x 6144 within 3 % either way, 15360 x 5120
        # level, 3584 x 5120 5.7 / 6.0 -> 6.2 / 7.0; K = 4096: 4096 x 4096 level, 12288 and 22016 wide 8 - 13 % and 3 - 13 % slower)
        return None
    if not mgemv_supported(K, nbits, group_size):
        return None
    if nbits in (2, 3) and mgemv_tiling(M, N, K, nbits, group_size) is not None:
        return None
    mt16 = -(-M // 16)
    if mt16 == 2:
        # 17 .. 32 rows (two activation tiles per wave, eight to eleven waves): measured against the GEMM kernel with
        # 32-row tiles, which serves long rows there otherwise: 4096 x 11008 19.4 -> 12.5 us, 4096 x 14336 23.8 -> 17.1;
        # level at K = 8192 (8192 x 8192 17.2 -> 16.7, 10240 x 8192 21.0 -> 20.5), slower on wide or very long layers
        # (57344 x 8192 67 -> 87, 8192 x 28672 45 -> 54): only narrow layers with long rows
        if nbits != 4 or not N or N > 4096 or K < 11008 or mgemv_tiling(M, N, K, nbits, group_size) is not None:
            return None
    chunk = 4 * (128 // plane_bits(nbits))
    if group_size % chunk and chunk % group_size:
        return None
    nchunk = K // chunk
    ch = max(1, KSPLIT_WAVE_K // chunk)
    ks = 2
    while ks <= 16:
        nb = -(-nchunk // ks)
        wk = -(-nb // ch)
        # (2 and 3 bits: the transposition buffers of sixteen waves do not fit the LDS; eight do)
        if wk <= 16 and mgemv_regs(mt16, ch, 1, nbits) <= mgemv_reg_limit(wk) and mgemv_lds_bytes(mt16, wk, ch, nbits) <= 160 * 1024:
            break
        ks *= 2
    if ks > 16 or (ks - 1) * nb >= nchunk or (wk - 1) * ch >= nb:
        return None
    return {"MT16": mt16, "WK": wk, "CH": ch, "PB": NUM_CUS // ks, "PF": 1, "KS": ks}


def mgemv_candidates(M, N, K, nbits, group_size):
    split = mgemv_ksplit_tiling(M, N, K, nbits, group_size)
    base = mgemv_tiling(M, N, K, nbits, group_size)
    if base is None:
        return [split] if split else []
    seen, out = set(), ([split] if split else [])
    nchunk = K // (4 * (128 // plane_bits(nbits)))

    def add(cfg):
        key = tuple(sorted(cfg.items()))
        ok = (cfg["WK"] <= 16 and cfg["WK"] * cfg["CH"] >= nchunk and (cfg["WK"] - 1) * cfg["CH"] < nchunk
              and cfg["CH"] <= nchunk
              and mgemv_regs(cfg["MT16"], cfg["CH"], cfg["PF"], nbits) <= mgemv_reg_limit(cfg["WK"])
              and mgemv_lds_bytes(cfg["MT16"], cfg["WK"], cfg["CH"], nbits) <= 160 * 1024)
        if ok and key not in seen:
            seen.add(key)
            out.append(cfg)

    add(base)
    for ch in (1, 2, 4, 8, 16):
        wk = -(-nchunk // ch)
        for pb in (NUM_CUS // 2, NUM_CUS, 2 * NUM_CUS):
            for pf in (1, 2, 4):
                add({"MT16": base["MT16"], "WK": wk, "CH": ch, "PB": pb, "PF": pf})
    return out


def mgemv_cfg_string(problem, t, nt_b):
    b = lambda x: "true" if x else "false"
    return (f"qf::MGemvCfg<{problem['NBITS']}, {problem['GS']}, {b(problem['SYM'])}, {problem['N']}, {problem['K']}, "
            f"{t['MT16']}, {t['WK']}, {t['CH']}, {t['PB']}, {t['PF']}, {b(nt_b)}"
            + (f", {t['KS']}>" if t.get("KS", 1) > 1 else ">"))


# --------------------------------------------------------------------------------------------
# Skinny MFMA regime (3 <= M <= 32): qf::SkinnyCfg (include/qf_skinny.hip.h) -- every load lands in
# fragment order, WK waves split K in steps of 128 packed bytes, SB tiles per batch, D stages in flight
# --------------------------------------------------------------------------------------------

def skinny_supported(K, nbits, group_size):
    if nbits not in (2, 4, 8) or not group_size or group_size <= 0:
        return False
    epl = 128 // nbits
    chunk, stepk = 4 * epl, 8 * epl
    if K % stepk or K % group_size or group_size % epl:
        return False
    if (group_size % stepk) if group_size >= stepk else (chunk % group_size):
        return False
    return (K // group_size) % (8 // nbits) == 0


SKINNY_MAX_M = 16
SKINNY_MAX_K = 16384


def skinny_preferred(M, K, nbits, group_size, N=None):
    """The streaming kernel takes the rows-of-16 problems whose activations the A-stationary kernel
    cannot keep in registers (K = 11008 or 14336 at 4 bits, K = 8192 or 11008 at 8 bits).  Measured at
    M = 4 .. 16 on 4096 x 11008: 10.7 .. 13.2 us against 13.9 .. 21.7 us for the kernels that served it
    before (8-bit: 17.4 against 28.6).  Every block streams all of the activations, M x K x 2 bytes:
    at K = 28672 that is twice the block's weight bytes and the GEMM kernel wins (49 against 109 us),
    as it does above 16 rows.  Between 16384 and 20480 it still wins where every block has a single tile of
    16 columns while 32-column GEMM tiles would leave half of the CUs idle (3584 x 18944 at 4 bits: 20.6
    against 32.0 us)."""
    if not (MGEMV_MIN_M <= M <= SKINNY_MAX_M):
        return False
    if K > SKINNY_MAX_K and not (nbits == 4 and K <= 20480 and N is not None and 0 < N <= 16 * NUM_CUS):
        return False
    return skinny_tiling(M, 16 * NUM_CUS, K, nbits, group_size) is not None


def skinny_regs(cfg, nbits, spw):
    """Rough VGPR need of qf::skinny_kernel: D stages (coalesced activation rows unless resident,
    packed words), the activation fragments in use (all the wave's steps when AST), the batch's
    scales and zero-points twice, accumulators, ~48 of addresses and temporaries."""
    stepk = 8 * (128 // nbits)
    a_step = cfg["MT16"] * stepk // 8                  # registers of one activation step (16 rows x STEPK halves / 64 lanes)
    stage = (0 if cfg["AST"] else a_step) + cfg["SB"] * 8
    quant = 2 * cfg["SB"] * 2 * spw
    frags = spw * a_step if cfg["AST"] else a_step
    return cfg["D"] * stage + frags + quant + cfg["SB"] * cfg["MT16"] * 8 + 48


def skinny_lds_bytes(cfg, nbits):
    stepk = 8 * (128 // nbits)
    return 2 * cfg["WK"] * cfg["SB"] * cfg["MT16"] * 1024 + cfg["WK"] * cfg["MT16"] * 16 * (stepk * 2 + 16)


def skinny_valid(cfg, N, K, nbits, group_size):
    import math
    if not skinny_supported(K, nbits, group_size):
        return False
    mt16, wk, sb, d = cfg["MT16"], cfg["WK"], cfg["SB"], cfg["D"]
    nstep = K // (8 * (128 // nbits))
    spw = -(-nstep // wk)
    if not (1 <= mt16 <= 2 and 1 <= wk <= 16 and 1 <= sb <= 8 and 1 <= d <= 4):
        return False
    if (wk - 1) * spw >= nstep or math.lcm(spw, d) > 32:
        return False
    if skinny_lds_bytes(cfg, nbits) > 160 * 1024:
        return False
    return skinny_regs(cfg, nbits, spw) <= min(512, 512 // -(-wk // 4))


def skinny_tiling(M, N, K, nbits, group_size, **pins):
    """Default tiling (None if the kernel does not cover the problem), from on-device sweeps at
    M = 16: eight waves per block; one tile per batch unless a block sweeps four or more; the
    activation fragments stay resident when a block has several batches and they fit; two stages
    in flight."""
    if not skinny_supported(K, nbits, group_size) or M > 32:
        return None
    mt16 = -(-M // 16)
    nstep = K // (8 * (128 // nbits))
    nt = -(-N // 16)
    slots = -(-nt // min(nt, NUM_CUS))
    best = None
    for wk in range(min(8, nstep), 0, -1):
        spw = -(-nstep // wk)
        if (wk - 1) * spw >= nstep:
            continue
        waste = (wk * spw - nstep) / nstep
        for sb in ((2, 1) if slots >= 4 else (1,)):
            nbatch = -(-slots // sb)
            for ast in ((1, 0) if nbatch > 1 else (0,)):
                for d in (2, 1):
                    cfg = {"MT16": mt16, "WK": wk, "SB": sb, "D": d, "AST": ast, "PB": NUM_CUS}
                    if not skinny_valid(cfg, N, K, nbits, group_size):
                        continue
                    key = (waste > 0.13, -wk, -ast, -sb, -d)
                    if best is None or key < best[0]:
                        best = (key, cfg)
    if best is None:
        return None
    cfg = best[1]
    cfg.update(pins)
    return cfg


def skinny_candidates(M, N, K, nbits, group_size):
    base = skinny_tiling(M, N, K, nbits, group_size)
    if base is None:
        return []
    seen, out = set(), []

    def add(cfg):
        key = tuple(sorted(cfg.items()))
        if key not in seen and skinny_valid(cfg, N, K, nbits, group_size):
            seen.add(key)
            out.append(cfg)

    add(base)
    for wk in (base["WK"], 8, 7, 6, 4):
        for sb in (1, 2):
            for d in (1, 2, 3):
                for ast in (0, 1):
                    add({"MT16": base["MT16"], "WK": wk, "SB": sb, "D": d, "AST": ast, "PB": NUM_CUS})
    return out


def skinny_cfg_string(problem, t, nt_b):
    b = lambda x: "true" if x else "false"
    return (f"qf::SkinnyCfg<{problem['NBITS']}, {problem['GS']}, {b(problem['SYM'])}, {problem['N']}, {problem['K']}, "
            f"{t['MT16']}, {t['WK']}, {t['SB']}, {t['D']}, {b(t['AST'])}, {t['PB']}, {b(nt_b)}>")


# --------------------------------------------------------------------------------------------
# Large-M GEMM regime (qf::GemmCfg, include/qf_gemm.hip.h): weights dequantised into MFMA
# fragment registers, activations loaded straight into LDS (PA tiles ahead), WK wave groups
# splitting K inside a block
# --------------------------------------------------------------------------------------------
GEMM_BK = 64


def gemm_lds_bytes(cfg, nbits=4):
    bm, nt32, wn, wk = cfg["BM"], cfg["NT32"], cfg["WN"], cfg["WK"]
    bn = 32 * nt32 * wn
    lds_a = wk * cfg["PA"] * bm * GEMM_BK * 2
    lds_red = (wk - 1) * bm * bn * 4
    return max(lds_a, lds_red) + wk * wn * 32 * nt32 * (144 + (80 if nbits == 3 else 0))


def gemm_regs(cfg):
    """Rough VGPR need of one lane: accumulators, two sets of activation fragments, the weight
    super ring, plus ~50 of addresses and dequantisation temporaries (compiled: 192 for 64 x 32 wave
    tiles with two groups, 250 for 256 x 32 ones).  A SIMD has 512 per lane to
    share between the waves a block puts on it (spills are ruinous)."""
    mt32, nt32 = cfg["BM"] // 32, cfg["NT32"]
    ua = max(1, cfg["BM"] * 8 // (64 * cfg["WN"]))
    frag_sets = 2 if mt32 <= 4 else 0.25               # tall tiles keep one k-step of fragments, not two tiles
    return int(mt32 * nt32 * 16 + frag_sets * mt32 * 16 + 2 * nt32 * 20 + ua + 50)


def gemm_valid(cfg, K, nbits, group_size):
    """Mirror of the static checks in gemm_launch (qf_gemm.hip.h)."""
    if nbits not in (2, 3, 4, 8):
        return False
    pb, zfb = plane_bits(nbits), (4 if nbits == 3 else nbits)
    supk = 1024 // pb
    bm, nt32, wn, wk, pa = (cfg[k] for k in ("BM", "NT32", "WN", "WK", "PA"))
    if bm <= 0 or bm % 32 or min(nt32, wn, wk) < 1 or 64 * wn * wk > 1024:
        return False
    # K: whole 64-element iterations and at least one 128-byte window of the main plane; a partial last
    # window must be whole 16-byte units in every plane
    if K % 64 or K < supk or ((K % supk) * pb // 8) % (32 if nbits == 3 else 16):
        return False
    if K % group_size or group_size % 32:
        return False
    if (group_size < supk and supk % group_size) or (group_size > supk and group_size % supk):
        return False
    ngs = max(1, supk // group_size)
    if ngs > 8 or ngs * zfb > 32:
        return False
    # (asymmetric weights also need K/GS to fill whole zero-point bytes: a property of the packed tensors,
    # checked where they are built and again by the launcher, not a tiling matter -- symmetric ones do not)
    if not 3 <= pa <= 12:
        return False
    if (bm // 32) * nt32 * 16 > 256:
        return False
    if gemm_regs(cfg) * max(1, 64 * wn * wk // 256) > 512:
        return False
    return gemm_lds_bytes(cfg, nbits) <= 160 * 1024


def gemm_supported(K, nbits, group_size):
    probe = {"BM": 64, "NT32": 1, "WN": 4, "WK": 1, "PA": 3}
    return gemm_valid(probe, K, nbits, group_size)


_GEMM_TUNED = None


def gemm_tuned(M, N, K, nbits, group_size):
    """The winner of the on-device sweep over ``gemm_candidates`` for this exact problem, where the sweep was run
    and beat the model below by 3 % or more (``gemm_tuned_gfx950.json`` beside this file: the reference times its
    candidates at every first construction, qfunc.py:110-131; here that was done once for the reference's own
    shape list at M = 32 .. 256, W4 g128).  None for any other problem."""
    global _GEMM_TUNED
    if _GEMM_TUNED is None:
        import json
        import os
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_tuned_gfx950.json")
        try:
            with open(path) as f:
                _GEMM_TUNED = json.load(f)
        except FileNotFoundError:
            _GEMM_TUNED = {}
    cfg = _GEMM_TUNED.get(f"{nbits}-{M}-{N}-{K}-{group_size}")
    return dict(cfg) if cfg is not None and gemm_valid(cfg, K, nbits, group_size) else None


def gemm_tiling(M, N, K, nbits, group_size, **pins):
    """Default GEMM tiling: the swept winner where there is one (``gemm_tuned``), else a small cost model fitted to
    on-device sweeps: a launch takes
    ceil(blocks / CUs) rounds of one tile's work, and a tile costs its area plus a fixed overhead
    (pipeline fill, reduction, barriers) worth about 2048 outputs.  It reproduces the measured
    winners: 64 x 128 tiles on 8192-wide, 128 x 128 on 10240-wide (160 tiles in one round beat 320
    in two) and 256 x 256 on 57344-wide layers at M = 256; 32 x 32 ... 64 x 64 tiles for M <= 128."""
    import math
    cfg = gemm_tuned(M, N, K, nbits, group_size)
    if cfg is not None:
        cfg.update(pins)
        return cfg
    if M >= 512:
        cfg = _gemm_tiling_many_rows(M, N, K, nbits, group_size)
        if cfg is not None:
            cfg.update(pins)
            return cfg
    best = None
    for bm in (256, 128, 64, 32):
        if bm >= 2 * M and bm > 32:
            continue
        # 256-row tiles: eight waves side by side (a 256 x 256 block tile, every weight dequantised
        # once); measured 250 against 300 us on 57344 x 8192 at M = 256
        # any number of waves along N: the count that deals the columns to the 256 CUs in whole rounds wins (57344
        # columns are 256 tiles of 7 x 32: 230 against 269 us for 224 tiles of 8 x 32 at M = 256; 22016 x 4096 at
        # M = 256: 58.6 us for six waves against 67.1 for 128 x 256 tiles)
        # (32-row tiles keep 4 / 2 / 1: with the odd counts the model over-picked them -- mean regret over the 124
        # swept cells 1.032 against 1.017, worst 1.36 against 1.23)
        for wn in ((8, 7, 6, 5) if bm == 256 else ((4, 7, 6, 5, 3, 2, 1) if bm >= 64 else (4, 2, 1))):
            for nt32 in ((1, 2) if (bm, wn) == (128, 4) else (1,)):
                bn = 32 * wn * nt32
                blocks = -(-N // bn) * -(-M // bm)
                rounds = -(-blocks // NUM_CUS)
                cost = rounds * (bm * bn + 2048)
                key = (cost, abs(math.log2(bm / bn)), -bn)
                if best is None or key < best[0]:
                    best = (key, bm, wn, nt32, blocks)
    _, bm, wn, nt32, blocks = best
    # with at most one block per CU the K axis is split over wave groups inside the block, so
    # that every SIMD still holds two waves (one dequantises while the other multiplies)
    # (no more than four groups: eight groups of one wave leave LDS for three activation tiles per group only and
    # measured slower than four groups with four tiles, 20.6 against 18.3 us on 8192 x 8192 at M = 32, 23.0 against
    # 21.0 on 4096 x 11008 at M = 64)
    wk = max(1, min(4, 8 // wn)) if blocks <= NUM_CUS else 1
    if bm >= 128:
        wk = 1                                        # 128-row tiles in two wave groups spill (six waves of 128 x 32: 85 against 38 us)
    nsup = -(-K // (1024 // plane_bits(nbits)))
    wk = max(1, min(wk, nsup))
    # 128 x 256 block tiles of four 128 x 64 waves: three activation tiles in flight measured 128.7 against 156.7 us
    # for four on 57344 x 8192 at M = 128 and the same on 22016 x 4096 at M = 256
    pa_first = 3 if (bm, nt32, wn) == (128, 2, 4) else 4
    pa = pa_first
    while not gemm_valid({"BM": bm, "NT32": nt32, "WN": wn, "WK": wk, "PA": pa}, K, nbits, group_size):
        if pa == 4:
            pa = 3                                    # one activation tile less in LDS
        elif wk > 1:
            wk, pa = wk // 2, pa_first
        else:
            break
    cfg = {"BM": bm, "NT32": nt32, "WN": wn, "WK": wk, "PA": pa}
    cfg.update(pins)
    return cfg


def gemm_tiling_model(M, N, K, nbits, group_size):
    """The cost model's choice alone (what ``gemm_tiling`` returns for a problem that was never swept)."""
    global _GEMM_TUNED
    saved, _GEMM_TUNED = _GEMM_TUNED, {}
    try:
        return gemm_tiling(M, N, K, nbits, group_size)
    finally:
        _GEMM_TUNED = saved


def _gemm_tiling_many_rows(M, N, K, nbits, group_size):
    """M >= 512 (prefill): several rounds of blocks, one group per block.  Fitted to a sweep over
    M = 512 .. 2048 on eight Llama shapes: a tile costs its area plus an overhead worth 6300 outputs
    (per round at K = 8192: 48 us for 64 x 128, 85 for 128 x 128, 140 for 128 x 256, 250 for 256 x 256);
    rounds overlap, so a launch costs its exact number of rounds plus 60 % of the rounding-up, and a
    single partial round runs faster than a full one (0.6 + 0.4 x the fraction of CUs with a block;
    with 0.75 + 0.25 the model kept 128 x 128 tiles in 2.5 rounds on 10240 x 8192 at M = 1024, 294 us,
    where 160 tiles of 256 x 256 take 224 us, and on 22016 x 4096 at M = 512, 146 against 123 us).
    Picks within 4 % of the best of the sweep on 22 of 24 cells (before: 17; worst case 1.35x -> 1.16x).  None when the launch is a
    single round: the small-M model, which splits K over wave groups, serves those.  (Wave counts of 3, 5, 6, 7
    along N, which pay for single-round launches, were measured here too: within 2 % of the eight-wave tiles at best
    over several rounds, and the round model mis-ranks them by up to 12 %; not offered.)"""
    best = None
    for bm, nt32, wn in ((256, 1, 8), (128, 2, 4), (128, 1, 4), (64, 1, 4)):
        cfg = {"BM": bm, "NT32": nt32, "WN": wn, "WK": 1, "PA": 4 if bm <= 128 else 3}
        if not gemm_valid(cfg, K, nbits, group_size):
            continue
        bn = 32 * wn * nt32
        exact = (-(-N // bn) * -(-M // bm)) / NUM_CUS
        rounds = exact + 0.6 * (-(-exact // 1) - exact) if exact >= 1 else 0.6 + 0.4 * exact
        cost = rounds * (bm * bn + 6300)
        if best is None or cost < best[0]:
            best = (cost, cfg)
    if best is None or -(-N // 128) * -(-M // 64) <= NUM_CUS:
        return None                    # at most one round even of 64 x 128 tiles: the small-M model, which splits K over wave groups
    return best[1]


def gemm_candidates(M, N, K, nbits, group_size):
    seen, out = set(), []

    def add(cfg):
        key = tuple(sorted(cfg.items()))
        if key not in seen and gemm_valid(cfg, K, nbits, group_size):
            seen.add(key)
            out.append(cfg)

    add(gemm_tiling(M, N, K, nbits, group_size))
    for bm in (32, 64, 128, 256):
        if bm >= 2 * M and bm > 32:
            continue
        for nt32 in (1, 2):
            for wn in (1, 2, 3, 4, 5, 6, 7, 8):          # any count: 57344 columns are 256 tiles of 7 x 32, one per CU
                for wk in (1, 2, 4, 8):
                    for pa in (3, 4, 6):
                        add({"BM": bm, "NT32": nt32, "WN": wn, "WK": wk, "PA": pa})
    return out


def gemm_cfg_string(problem, t, nt_b):
    b = lambda x: "true" if x else "false"
    return (f"qf::GemmCfg<{problem['NBITS']}, {problem['GS']}, {b(problem['SYM'])}, {problem['N']}, {problem['K']}, "
            f"{t['BM']}, {t['NT32']}, {t['WN']}, {t['WK']}, {t['PA']}, {b(nt_b)}>")
