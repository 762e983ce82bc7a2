"""Checks on the generated ISA of a compiled object.

The GEMM kernel (include/qf_gemm.hip.h) publishes its activation tiles with ``s_waitcnt vmcnt(n)``, n being the
number of vector-memory loads the wave has issued since the tile's request -- a count made at compile time from
how many loads every K-iteration issues.  A wave's loads return in order, so the wait is right exactly when the
compiled code issues those loads, all of them, between the barriers the count assumes.  A compiler that drops or
merges loads whose results are unused (it did once, on a K loop with a single trip) makes the wait too weak: a tile
could be read before it has landed, silently and not on every run.  ``gemm_waits_hold`` re-counts the loads on the
ISA; the JIT calls it for every GEMM object and rebuilds the object with a full drain if the count does not hold.
"""
import re

_WAIT = re.compile(r"s_waitcnt vmcnt\((\d+)\) lgkmcnt\(0\)")


def gemm_waits_hold(isa: str, pa: int):
    """(ok, detail) for the ISA text of one GEMM translation unit compiled with PA activation tiles in flight.

    Between two of the kernel's explicit waits lies one K-iteration.  A wait that allows n loads in flight must be
    preceded by exactly n vector-memory loads in the last PA - 2 iterations.  At least two waits must be checkable
    (the unrolled K loop has at least two iterations)."""
    loads_in_segment, segments, checked = 0, [], 0
    for line in isa.splitlines():
        line = line.strip()
        if line.startswith(("global_load", "buffer_load")):
            loads_in_segment += 1
            continue
        m = _WAIT.match(line)
        if not m:
            continue
        allowed = int(m.group(1))
        segments.append(loads_in_segment)
        loads_in_segment = 0
        if allowed == 0:
            segments = []                      # a full drain: nothing older is in flight
        elif len(segments) >= pa - 2:
            have = sum(segments[-(pa - 2):])
            if have != allowed:
                return False, f"a wait allows {allowed} loads in flight but the last {pa - 2} iterations issue {have} ({segments})"
            checked += 1
    if checked < 2:
        return False, f"only {checked} counted waits found"
    return True, f"{checked} counted waits match the loads issued"
