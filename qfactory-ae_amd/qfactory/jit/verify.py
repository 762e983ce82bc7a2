"""Checks on the generated ISA of a compiled object.

The GEMM kernel (include/qf_gemm.hip.h) publishes its activation tiles with ``s_waitcnt vmcnt(n)``, n being the
number of vector-memory loads the wave has issued since the tile's request -- a count made at compile time from
how many loads every K-iteration issues.  A wave's loads return in order, so the wait is right exactly when the
compiled code issues at least those n loads behind the request, on every path.  A compiler that drops or merges
loads whose results are unused (it did once, on a K loop with a single trip) makes the wait too weak: a tile could
be read before it has landed, silently and not on every run.  ``gemm_waits_hold`` re-counts the loads on the ISA,
along the control flow; the JIT calls it for every GEMM object and rebuilds the object with a full drain per
K-iteration if the count does not hold.
"""
import re

_WAIT = re.compile(r"s_waitcnt vmcnt\((\d+)\) lgkmcnt\(0\)")
_LABEL = re.compile(r"^(\.LBB\d+_\d+):")
_BRANCH = re.compile(r"^(s_branch|s_cbranch_\w+)\s+(\.LBB\d+_\d+)")
_LOADS = ("global_load", "buffer_load", "flat_load", "scratch_load")


def _blocks_of(isa):
    """Basic blocks of the (single) kernel in the listing: name -> (events, successors); an event is 'L' (a
    vector-memory load) or ('W', n) (one of the kernel's explicit waits).  The entry block is named 'entry'."""
    blocks, order = {}, []
    name, events, succ, open_block = "entry", [], [], False
    started = False

    def close(fallthrough_to=None):
        nonlocal events, succ
        if fallthrough_to is not None:
            succ.append(fallthrough_to)
        blocks[name] = (events, succ)
        order.append(name)
        events, succ = [], []

    for raw in isa.splitlines():
        line = raw.strip()
        if not started:
            if re.match(r"^_Z\w+:", raw):                               # the kernel's own label
                started, open_block = True, True
            continue
        if line.startswith(".Lfunc_end"):
            break
        m = _LABEL.match(line)
        if m:
            if open_block:
                close(fallthrough_to=m.group(1))
            name, open_block = m.group(1), True
            continue
        if not line or line[0] in ".;":
            continue
        if not open_block:                                            # code after an unconditional branch without a label
            name, open_block = f"anon{len(order)}", True
        if line.startswith(_LOADS):
            events.append("L")
            continue
        w = _WAIT.match(line)
        if w:
            events.append(("W", int(w.group(1))))
            continue
        b = _BRANCH.match(line)
        if b:
            succ.append(b.group(2))
            if b.group(1) == "s_branch":
                close()
                open_block = False
            else:                                                     # a conditional branch ends its block too
                after = f"after{len(order)}"
                close(fallthrough_to=after)
                name = after
            continue
        if line.startswith("s_endpgm"):
            close()
            open_block = False
    if open_block:
        close()
    return blocks


def gemm_waits_hold(isa: str, pa: int):
    """(ok, detail) for the ISA text of one GEMM translation unit compiled with PA activation tiles in flight.

    Between two of the kernel's explicit waits lies one K-iteration.  A wait that allows n loads in flight publishes
    a tile requested PA - 2 iterations earlier, so on every control-flow path that leads to it the wave must have
    issued at least n vector-memory loads in those PA - 2 iterations (a path that crosses a full drain, vmcnt(0), is
    safe: nothing older is in flight).  At least two counted waits must be found."""
    blocks = _blocks_of(isa)
    if not blocks:
        return False, "no kernel found in the listing"
    preds = {b: [] for b in blocks}
    for b, (_, succ) in blocks.items():
        for s in succ:
            if s in preds:
                preds[s].append(b)
    back = pa - 2
    checked, exact = 0, True
    budget = [200000]

    def min_loads(block, upto, waits_left):
        """Fewest loads issued on any path ending just before event index `upto` of `block`, going back over
        `waits_left` waits; None if every such path crosses a full drain first."""
        budget[0] -= 1
        if budget[0] < 0:
            raise RuntimeError("control flow too tangled to enumerate")
        events = blocks[block][0]
        count = 0
        for i in range(upto - 1, -1, -1):
            ev = events[i]
            if ev == "L":
                count += 1
            else:
                if ev[1] == 0:
                    return None
                waits_left -= 1
                if waits_left == 0:
                    return count
        best = None
        if not preds[block]:
            return None                                               # the kernel's entry: nothing older is in flight
        for p in preds[block]:
            r = min_loads(p, len(blocks[p][0]), waits_left)
            if r is not None and (best is None or r < best):
                best = r
        return None if best is None else count + best

    try:
        for b, (events, _) in blocks.items():
            for i, ev in enumerate(events):
                if ev == "L" or ev[1] == 0:
                    continue
                have = min_loads(b, i, back)
                if have is None:
                    continue                                          # only reachable right behind a full drain
                if have < ev[1]:
                    return False, (f"a wait in {b} allows {ev[1]} loads in flight but a path issues only {have} "
                                   f"in the {back} iterations before it")
                exact = exact and have == ev[1]
                checked += 1
    except RuntimeError as exc:
        return False, str(exc)
    if checked < 2:
        return False, f"only {checked} counted waits found"
    return True, f"{checked} counted waits hold on every path" + ("" if exact else " (some allow fewer loads than are issued)")
