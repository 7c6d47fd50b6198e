#!/usr/bin/env python3
"""Writes fast_schedules.h: the list of lengths that get a compile-time-schedule
tile kernel (fast_core.h) and the radix schedule of each.

Run by hand when the list changes:  python3 gen_fast_schedules.py > fast_schedules.h

A schedule has at most four passes with radices from RADICES.  Threads per
transform follow from the schedule exactly as the planner computes them for
the generic kernel (a thread holds at most REG_ELEMS complex values per pass),
so a plan made for a fast kernel can also run on the generic one.
"""
import itertools
import sys

REG_ELEMS = 16
RADICES = [16, 10, 9, 8, 7, 6, 5, 4, 3, 2]
MAX_N = 4096
SLICES = 8

# Threads per transform (single, double precision) where the default -- the fewest the
# register budget allows -- is not the fastest: measured on MI355X with batched
# unit-stride complex transforms of 2^24 (single) / 2^23 (double) points in total.
TUNED_TPT = {
    12: (4,4), 14: (2,2), 15: (5,5), 18: (3,3), 20: (4,4), 21: (3,3), 24: (6,6), 25: (5,5),
    27: (0,9), 28: (4,4), 30: (5,5), 35: (7,7), 36: (6,6), 40: (5,5), 42: (7,7), 48: (6,6),
    49: (7,7), 56: (8,8), 63: (9,9), 70: (10,10), 72: (9,9), 75: (15,15), 80: (8,8), 84: (12,12),
    98: (14,14), 105: (15,15), 108: (18,0), 125: (25,25), 126: (21,21), 140: (20,20), 147: (21,21),
    150: (30,30), 168: (24,24), 175: (35,35), 180: (30,30), 192: (24,24), 196: (28,28),
    210: (42,42), 216: (36,36), 224: (28,28), 225: (0,45), 240: (30,30), 245: (49,49),
    252: (42,42), 280: (56,56), 288: (48,48), 294: (49,49), 315: (63,63), 320: (40,40),
    324: (0,41), 336: (56,56), 343: (49,49), 360: (60,60), 375: (75,125), 378: (63,63),
    384: (48,64), 392: (56,56), 420: (70,70), 432: (0,72), 441: (63,63), 448: (64,64),
    450: (90,90), 486: (0,81), 490: (70,70), 504: (72,72), 525: (75,175), 540: (90,90),
    567: (81,81), 588: (84,84), 625: (125,125), 630: (90,90), 640: (80,0), 648: (81,81),
    686: (0,98), 700: (100,100), 720: (90,90), 735: (105,245), 750: (150,150), 768: (64,64),
    864: (144,144), 875: (175,175), 882: (147,147), 960: (160,160), 980: (140,245),
    1008: (144,144), 1029: (147,147), 1050: (210,210), 1080: (216,216), 1120: (160,160),
    1134: (189,189), 1152: (144,144), 1176: (168,168), 1225: (175,245), 1260: (252,252),
    1280: (128,128), 1344: (168,168), 1372: (196,196), 1400: (175,175), 1470: (210,210),
    1512: (252,252), 1568: (196,196), 1680: (210,210), 1715: (245,245), 1764: (252,252),
    1944: (243,243), 1960: (245,245), 2058: (343,343), 2240: (280,448), 2352: (392,392),
    2401: (343,343), 2430: (0,486), 2592: (324,324), 2646: (441,441), 2688: (224,224),
    2700: (450,450), 2744: (392,392), 2916: (486,486), 2940: (490,490), 3000: (500,500),
    3024: (504,504), 3072: (256,256), 3087: (441,441), 3136: (448,448), 3150: (450,450),
    3240: (405,405), 3402: (486,486), 3430: (490,490), 3528: (504,504), 3600: (450,450),
    4000: (0,500),
}
# pass schedules where the default (fewest passes, least lane work) is not the fastest
TUNED_SCHEDULE = {
    12: (4, 3), 15: (3, 5), 18: (6, 3), 20: (5, 4), 24: (4, 6), 30: (6, 5), 35: (5, 7),
    40: (4, 10), 42: (6, 7), 48: (8, 6), 56: (7, 8), 63: (7, 9), 70: (7, 10), 72: (8, 9),
    80: (5, 16), 90: (9, 10), 96: (6, 16), 112: (7, 16), 120: (10, 6, 2), 126: (3, 6, 7),
    144: (9, 16), 150: (6, 5, 5), 160: (10, 16), 162: (9, 6, 3), 175: (5, 5, 7), 180: (6, 6, 5),
    192: (8, 8, 3), 210: (5, 6, 7), 224: (8, 7, 4), 240: (8, 6, 5), 245: (5, 7, 7), 252: (6, 6, 7),
    270: (3, 9, 10), 280: (5, 7, 8), 288: (8, 6, 6), 294: (6, 7, 7), 300: (10, 6, 5),
    315: (5, 7, 9), 320: (8, 8, 5), 336: (8, 7, 6), 360: (6, 6, 10), 378: (6, 7, 9),
    384: (8, 8, 6), 392: (7, 7, 8), 400: (10, 8, 5), 420: (6, 7, 10), 432: (9, 8, 6),
    441: (7, 7, 9), 448: (8, 8, 7), 450: (5, 9, 10), 480: (10, 8, 6), 490: (7, 7, 10),
    504: (7, 8, 9), 540: (6, 9, 10), 560: (10, 8, 7), 567: (7, 9, 9), 576: (6, 6, 16),
    630: (7, 9, 10), 640: (10, 8, 8), 648: (8, 9, 9), 672: (6, 7, 16), 700: (7, 10, 10),
    720: (10, 9, 8), 750: (6, 5, 5, 5), 756: (3, 6, 6, 7), 768: (3, 16, 16), 784: (7, 7, 16),
    810: (9, 9, 10), 840: (10, 7, 6, 2), 864: (6, 9, 16), 875: (5, 5, 5, 7), 882: (3, 6, 7, 7),
    896: (7, 8, 16), 900: (9, 10, 10), 960: (6, 10, 16), 1008: (7, 9, 16), 1050: (7, 6, 5, 5),
    1080: (5, 6, 6, 6), 1120: (7, 10, 16), 1134: (2, 7, 9, 9), 1152: (8, 9, 16),
    1176: (7, 7, 6, 4), 1200: (10, 10, 6, 2), 1260: (5, 6, 6, 7), 1280: (5, 16, 16),
    1296: (9, 9, 16), 1344: (8, 8, 7, 3), 1350: (3, 5, 9, 10), 1440: (9, 10, 16),
    1458: (9, 9, 6, 3), 1500: (10, 6, 5, 5), 1512: (6, 6, 6, 7), 1536: (6, 16, 16),
    1568: (8, 7, 7, 4), 1600: (10, 10, 16), 1620: (9, 9, 5, 4), 1680: (8, 7, 6, 5),
    1728: (16, 9, 4, 3), 1764: (9, 7, 7, 4), 1792: (7, 16, 16), 1800: (10, 6, 6, 5),
    1890: (3, 7, 9, 10), 1920: (3, 5, 8, 16), 1944: (4, 6, 9, 9), 2016: (3, 6, 7, 16),
    2058: (6, 7, 7, 7), 2100: (10, 7, 6, 5), 2240: (8, 8, 7, 5), 2304: (9, 16, 16),
    2352: (8, 7, 7, 6), 2430: (9, 9, 6, 5), 2560: (10, 16, 16), 2592: (9, 9, 8, 4),
    2646: (6, 7, 7, 9), 2688: (3, 7, 8, 16), 2744: (7, 7, 7, 8), 2800: (10, 8, 7, 5),
    2916: (9, 9, 6, 6), 3024: (9, 8, 7, 6), 3072: (3, 4, 16, 16), 3087: (7, 7, 7, 9),
    3136: (8, 8, 7, 7), 3150: (5, 7, 9, 10), 3240: (4, 9, 9, 10), 3360: (10, 8, 7, 6),
    3402: (6, 7, 9, 9), 3456: (6, 6, 6, 16), 3584: (2, 7, 16, 16), 3600: (10, 10, 9, 4),
    3780: (6, 7, 9, 10), 3840: (3, 5, 16, 16), 3888: (9, 9, 8, 6), 3920: (10, 8, 7, 7),
    4032: (9, 8, 8, 7),
}

# --all-variants lists every candidate thread count of every length (a tuning build)
ALL_VARIANTS = "--all-variants" in sys.argv[1:]

POW2 = {2: (2,), 4: (4,), 8: (8,), 16: (16,), 32: (8, 4), 64: (16, 4), 128: (16, 8),
        256: (16, 16), 512: (16, 8, 4), 1024: (16, 16, 4), 2048: (16, 16, 8),
        4096: (16, 16, 16), 8192: (16, 16, 8, 4)}


def tpt(n, sched):
    t = 1
    for r in sched:
        slots = REG_ELEMS // r
        t = max(t, (n // r + slots - 1) // slots)
    return t


def lane_work(n, sched):
    """Butterfly-input slots over all lanes and passes, idle ones included."""
    t = tpt(n, sched)
    return t * sum(((n // r + t - 1) // t) * r for r in sched)


def best_schedule(n):
    best = None
    for npass in range(1, 5):
        for combo in itertools.combinations_with_replacement(RADICES, npass):
            prod = 1
            for r in combo:
                prod *= r
            if prod != n:
                continue
            t = tpt(n, combo)
            if t > 512:
                continue
            # fewer passes first, then the least lane work, then the larger radices
            key = (npass, lane_work(n, combo), tuple(-r for r in combo))
            if best is None or key < best[0]:
                best = (key, combo)
        if best is not None:
            break
    return best[1] if best else None


def tpt_candidates(n, sched):
    """Thread counts that change the butterflies per thread of some pass."""
    lo = tpt(n, sched)
    cand = set([lo])
    for r in sched:
        b = n // r
        for s_ in range(1, REG_ELEMS // r + 1):
            t = (b + s_ - 1) // s_
            if lo <= t <= 512:
                cand.add(t)
    return sorted(cand)


def all_schedules(n):
    """Every radix multiset (largest first) with the fewest passes."""
    found = []
    for npass in range(1, 5):
        for combo in itertools.combinations_with_replacement(RADICES, npass):
            prod = 1
            for r in combo:
                prod *= r
            if prod == n and tpt(n, combo) <= 512:
                found.append(combo)
        if found:
            break
    return sorted(found, key=lambda c: (lane_work(n, c), tuple(-r for r in c)))


def tuning_variants(n):
    """(schedule, threads) candidates of a tuning build, the default first."""
    out = []
    scheds = all_schedules(n)[:3]
    if scheds and len(scheds[0]) > 1:
        scheds.append(tuple(reversed(scheds[0])))
    for sc in scheds:
        cand = tpt_candidates(n, sc)
        keep = [cand[0]]
        b0 = n // sc[0]
        exact0 = [t for t in cand if b0 % t == 0]  # no idle lanes in the first pass
        for t in exact0[:2] + [cand[len(cand) // 2], cand[-1]]:
            if t not in keep:
                keep.append(t)
        for t in keep[:4]:
            if (sc, t) not in out:
                out.append((sc, t))
    return out


def smooth(n):
    for p in (2, 3, 5, 7):
        while n % p == 0:
            n //= p
    return n == 1


def main():
    rows = []
    for n in sorted(POW2):
        rows.append((n, TUNED_SCHEDULE.get(n, POW2[n]), 1))
    for n in range(3, MAX_N + 1):
        if n & (n - 1) == 0 or not smooth(n):
            continue
        s = TUNED_SCHEDULE.get(n) or best_schedule(n)
        if s:
            rows.append((n, s, 0))
    out = sys.stdout
    out.write("// fast_schedules.h -- generated by gen_fast_schedules.py, do not edit.\n")
    out.write("// FAST_SCHED(slice, all_modes, N, R0, R1, R2, R3, TPTF, TPTD): length N runs the passes R0..R3\n")
    out.write("// (1 = unused) with TPTF / TPTD threads per transform in single / double precision (0 = the\n")
    out.write("// fewest the register budget allows);\n")
    out.write("// all_modes = 1 builds the scalar and general vector variants besides the lean one;\n")
    out.write("// slice names the translation unit that instantiates the kernels.\n")
    out.write("#define FAST_SLICES %d\n" % SLICES)
    # spread by estimated compile cost: round-robin over rows sorted by size
    order = sorted(rows, key=lambda r: (-(3 if r[2] else 1) * r[0]))
    load = [0] * SLICES
    slice_of = {}
    for n, s, full in order:
        i = load.index(min(load))
        slice_of[n] = i
        load[i] += (3 if full else 1) * (n + 200)
    for n, s, full in sorted(rows):
        if ALL_VARIANTS:
            variants = [(sc, t, t) for sc, t in tuning_variants(n)]
        else:
            tf, td = TUNED_TPT.get(n, (0, 0))
            variants = [(s, tf, td)]
        for sc, tf, td in variants:
            r = list(sc) + [1] * (4 - len(sc))
            out.write("FAST_SCHED(%d, %d, %d, %d, %d, %d, %d, %d, %d)\n"
                      % (slice_of[n], full, n, r[0], r[1], r[2], r[3], tf, td))
    sys.stderr.write("%d lengths\n" % len(rows))


if __name__ == "__main__":
    main()
