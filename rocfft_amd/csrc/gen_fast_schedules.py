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
RADICES = [16, 13, 11, 10, 9, 8, 7, 6, 5, 4, 3, 2]
MAX_N = 4096
# Longer lengths (prime factors up to 5) that one workgroup of up to 1024 threads transforms
# in LDS in single precision; double precision where 512 threads and 160 KB of LDS suffice.
WIDE_LENGTHS = [4320, 4374, 4500, 4608, 4800, 4860, 5000, 5120, 5184, 5400, 5760, 5832, 6000, 6144, 6400,
                6480, 6561, 6912, 7200, 7290, 7680, 7776, 8000, 8100, 8640, 9000, 9216, 9600, 10000, 10240,
                12288, 16384]
LDS_BYTES = 160 * 1024
SLICES = 8

# Threads per transform (single, double precision) where the default -- the fewest the
# register budget allows -- is not the fastest: measured on MI355X with batched
# unit-stride complex transforms of 2^24 (single) / 2^23 (double) points in total.
TUNED_TPT = {
    12: (4,4), 14: (2,2), 15: (5,5), 18: (3,3), 20: (4,4), 21: (3,3), 22: (0,4), 24: (6,6),
    25: (5,5), 27: (0,9), 28: (4,4), 30: (5,5), 35: (7,7), 36: (6,6), 40: (5,5), 42: (7,7),
    48: (6,6), 49: (7,7), 55: (11,11), 56: (8,8), 63: (9,9), 70: (10,10), 72: (9,9), 75: (15,15),
    77: (11,11), 78: (13,13), 80: (8,8), 84: (12,12), 88: (11,11), 98: (14,14), 105: (15,15),
    108: (18,0), 125: (25,25), 126: (21,21), 132: (0,22), 140: (20,20), 147: (21,21), 150: (30,30),
    168: (24,24), 175: (35,35), 180: (30,30), 192: (24,24), 196: (28,28), 198: (22,22),
    210: (42,42), 216: (36,36), 224: (28,28), 225: (0,45), 234: (26,26), 240: (30,30),
    245: (49,49), 252: (42,42), 275: (28,0), 280: (56,56), 286: (48,48), 288: (48,48),
    294: (49,49), 315: (63,63), 320: (40,40), 324: (0,41), 336: (56,56), 343: (49,49),
    360: (60,60), 363: (0,61), 375: (75,125), 378: (63,63), 384: (48,64), 385: (0,77),
    390: (39,39), 392: (56,56), 396: (0,66), 420: (70,70), 429: (0,72), 432: (0,72), 440: (55,55),
    441: (63,63), 448: (64,64), 450: (90,90), 462: (0,77), 486: (0,81), 490: (70,70), 504: (72,72),
    507: (0,57), 525: (75,175), 539: (77,77), 540: (90,90), 546: (0,91), 567: (81,81), 572: (0,72),
    585: (0,117), 588: (84,84), 594: (99,99), 605: (61,0), 616: (88,88), 624: (52,52),
    625: (125,125), 630: (90,90), 640: (80,0), 648: (81,81), 660: (110,110), 686: (0,98),
    693: (99,99), 700: (100,100), 702: (117,117), 715: (72,72), 720: (90,90), 726: (0,121),
    735: (105,245), 750: (150,150), 768: (64,64), 770: (110,110), 780: (130,130), 792: (99,99),
    819: (117,117), 825: (0,138), 845: (0,85), 858: (0,143), 864: (144,144), 875: (175,175),
    880: (110,110), 882: (147,147), 910: (0,130), 924: (154,154), 936: (117,117), 960: (160,160),
    968: (121,121), 975: (0,109), 980: (140,245), 1001: (0,143), 1008: (144,144), 1014: (0,169),
    1029: (147,147), 1040: (104,104), 1050: (210,210), 1078: (0,154), 1080: (216,216),
    1120: (160,160), 1134: (189,189), 1144: (143,143), 1152: (144,144), 1155: (0,165),
    1176: (168,168), 1188: (0,198), 1225: (175,245), 1232: (176,176), 1260: (252,252),
    1280: (128,128), 1320: (165,165), 1344: (168,168), 1372: (196,196), 1400: (175,175),
    1408: (176,176), 1452: (182,182), 1456: (0,208), 1470: (210,210), 1512: (252,252),
    1568: (196,196), 1617: (0,231), 1638: (182,182), 1664: (208,208), 1680: (210,210),
    1694: (0,242), 1715: (245,245), 1716: (215,215), 1764: (252,252), 1815: (0,202),
    1848: (231,231), 1911: (0,213), 1944: (243,243), 1960: (245,245), 1980: (220,220),
    2002: (0,501), 2058: (343,343), 2145: (239,239), 2178: (242,242), 2240: (280,448),
    2340: (234,234), 2352: (392,392), 2401: (343,343), 2430: (0,486), 2457: (0,410),
    2475: (495,495), 2574: (0,429), 2592: (324,324), 2640: (440,440), 2646: (441,441),
    2673: (446,0), 2688: (224,224), 2700: (450,450), 2730: (455,455), 2744: (392,392),
    2860: (477,477), 2904: (484,484), 2916: (486,486), 2940: (490,490), 2970: (495,495),
    3000: (500,500), 3003: (501,501), 3024: (504,504), 3025: (303,0), 3042: (0,507),
    3072: (256,256), 3080: (440,440), 3087: (441,441), 3136: (448,448), 3146: (394,394),
    3150: (450,450), 3240: (405,405), 3276: (468,468), 3300: (367,367), 3380: (423,423),
    3388: (484,484), 3402: (486,486), 3430: (490,490), 3432: (429,429), 3465: (495,495),
    3520: (440,440), 3528: (504,504), 3549: (507,507), 3564: (446,446), 3575: (358,358),
    3600: (450,450), 3630: (404,404), 3640: (455,455), 3718: (465,465), 3872: (484,484),
    3900: (434,434), 3960: (495,495), 3993: (0,444), 4000: (0,500), 4004: (501,501),
    4056: (507,507),
}
# pass schedules where the default (fewest passes, least lane work) is not the fastest
TUNED_SCHEDULE = {
    16384: (16, 16, 4, 16),
    12: (4, 3), 15: (3, 5), 18: (6, 3), 20: (5, 4), 24: (4, 6), 30: (6, 5), 35: (5, 7),
    40: (4, 10), 42: (6, 7), 48: (8, 6), 55: (5, 11), 56: (7, 8), 63: (7, 9), 70: (7, 10),
    72: (8, 9), 77: (7, 11), 78: (6, 13), 80: (5, 16), 88: (8, 11), 90: (9, 10), 96: (6, 16),
    99: (9, 11), 110: (10, 11), 112: (7, 16), 117: (9, 13), 120: (10, 6, 2), 126: (3, 6, 7),
    130: (10, 13), 143: (11, 13), 144: (9, 16), 150: (6, 5, 5), 156: (2, 6, 13), 160: (10, 16),
    162: (9, 6, 3), 175: (5, 5, 7), 176: (11, 16), 180: (6, 6, 5), 192: (8, 8, 3), 198: (3, 6, 11),
    208: (13, 16), 210: (5, 6, 7), 220: (2, 10, 11), 224: (8, 7, 4), 234: (3, 6, 13),
    240: (8, 6, 5), 245: (5, 7, 7), 252: (6, 6, 7), 260: (2, 10, 13), 270: (3, 9, 10),
    280: (5, 7, 8), 288: (8, 6, 6), 294: (6, 7, 7), 297: (3, 9, 11), 300: (10, 6, 5),
    312: (4, 6, 13), 315: (5, 7, 9), 320: (8, 8, 5), 330: (11, 6, 5), 336: (8, 7, 6),
    351: (3, 9, 13), 352: (11, 8, 4), 360: (6, 6, 10), 378: (6, 7, 9), 384: (8, 8, 6),
    390: (5, 6, 13), 392: (7, 7, 8), 400: (10, 8, 5), 416: (13, 8, 4), 420: (6, 7, 10),
    432: (9, 8, 6), 440: (4, 10, 11), 441: (7, 7, 9), 448: (8, 8, 7), 450: (5, 9, 10),
    468: (6, 6, 13), 480: (10, 8, 6), 490: (7, 7, 10), 504: (7, 8, 9), 528: (11, 8, 6),
    539: (7, 7, 11), 540: (6, 9, 10), 550: (5, 10, 11), 560: (10, 8, 7), 567: (7, 9, 9),
    576: (6, 6, 16), 616: (7, 8, 11), 624: (3, 13, 16), 630: (7, 9, 10), 640: (10, 8, 8),
    648: (8, 9, 9), 650: (5, 10, 13), 660: (6, 10, 11), 672: (6, 7, 16), 693: (7, 9, 11),
    700: (7, 10, 10), 704: (11, 8, 8), 720: (10, 9, 8), 750: (6, 5, 5, 5), 756: (3, 6, 6, 7),
    768: (3, 16, 16), 770: (7, 10, 11), 780: (6, 10, 13), 784: (7, 7, 16), 792: (8, 9, 11),
    810: (9, 9, 10), 819: (7, 9, 13), 832: (13, 8, 8), 840: (10, 7, 6, 2), 864: (6, 9, 16),
    875: (5, 5, 5, 7), 880: (8, 10, 11), 882: (3, 6, 7, 7), 891: (9, 9, 11), 896: (7, 8, 16),
    900: (9, 10, 10), 924: (2, 6, 7, 11), 936: (8, 9, 13), 960: (6, 10, 16), 968: (8, 11, 11),
    990: (9, 10, 11), 1008: (7, 9, 16), 1040: (5, 13, 16), 1050: (7, 6, 5, 5), 1053: (9, 9, 13),
    1080: (5, 6, 6, 6), 1089: (9, 11, 11), 1092: (2, 6, 7, 13), 1100: (10, 10, 11),
    1120: (7, 10, 16), 1134: (2, 7, 9, 9), 1144: (8, 11, 13), 1152: (8, 9, 16), 1170: (9, 10, 13),
    1176: (7, 7, 6, 4), 1200: (10, 10, 6, 2), 1210: (10, 11, 11), 1232: (7, 11, 16),
    1248: (6, 13, 16), 1260: (5, 6, 6, 7), 1280: (5, 16, 16), 1287: (9, 11, 13), 1296: (9, 9, 16),
    1300: (10, 10, 13), 1320: (2, 6, 10, 11), 1344: (8, 8, 7, 3), 1350: (3, 5, 9, 10),
    1404: (3, 6, 6, 13), 1408: (8, 11, 16), 1430: (10, 11, 13), 1440: (9, 10, 16),
    1458: (9, 9, 6, 3), 1485: (3, 5, 9, 11), 1500: (10, 6, 5, 5), 1512: (6, 6, 6, 7),
    1521: (9, 13, 13), 1536: (6, 16, 16), 1540: (2, 7, 10, 11), 1560: (13, 8, 5, 3),
    1568: (8, 7, 7, 4), 1573: (11, 11, 13), 1584: (9, 11, 16), 1600: (10, 10, 16),
    1620: (9, 9, 5, 4), 1638: (3, 6, 7, 13), 1650: (3, 5, 10, 11), 1664: (8, 13, 16),
    1680: (8, 7, 6, 5), 1690: (10, 13, 13), 1728: (16, 9, 4, 3), 1760: (10, 11, 16),
    1764: (9, 7, 7, 4), 1782: (11, 9, 6, 3), 1792: (7, 16, 16), 1800: (10, 6, 6, 5),
    1820: (13, 10, 7, 2), 1848: (4, 6, 7, 11), 1859: (11, 13, 13), 1872: (9, 13, 16),
    1890: (3, 7, 9, 10), 1920: (3, 5, 8, 16), 1936: (11, 11, 16), 1944: (4, 6, 9, 9),
    1980: (11, 10, 6, 3), 2016: (3, 6, 7, 16), 2028: (2, 6, 13, 13), 2058: (6, 7, 7, 7),
    2079: (3, 7, 9, 11), 2080: (10, 13, 16), 2100: (10, 7, 6, 5), 2106: (13, 9, 6, 3),
    2112: (11, 8, 6, 4), 2178: (3, 6, 11, 11), 2184: (4, 6, 7, 13), 2200: (2, 10, 10, 11),
    2240: (8, 8, 7, 5), 2288: (11, 13, 16), 2304: (9, 16, 16), 2310: (11, 7, 6, 5),
    2340: (5, 6, 6, 13), 2352: (8, 7, 7, 6), 2420: (2, 10, 11, 11), 2430: (9, 9, 6, 5),
    2464: (11, 8, 7, 4), 2496: (2, 6, 13, 16), 2560: (10, 16, 16), 2592: (9, 9, 8, 4),
    2600: (13, 8, 5, 5), 2640: (11, 10, 8, 3), 2646: (6, 7, 7, 9), 2688: (3, 7, 8, 16),
    2704: (13, 13, 16), 2730: (13, 10, 7, 3), 2744: (7, 7, 7, 8), 2750: (5, 5, 10, 11),
    2800: (10, 8, 7, 5), 2808: (6, 6, 6, 13), 2816: (11, 16, 16), 2912: (13, 8, 7, 4),
    2916: (9, 9, 6, 6), 3024: (9, 8, 7, 6), 3072: (3, 4, 16, 16), 3087: (7, 7, 7, 9),
    3136: (8, 8, 7, 7), 3150: (5, 7, 9, 10), 3159: (3, 9, 9, 13), 3168: (11, 8, 6, 6),
    3240: (4, 9, 9, 10), 3250: (5, 5, 10, 13), 3267: (3, 9, 11, 11), 3276: (13, 9, 7, 4),
    3328: (13, 16, 16), 3360: (10, 8, 7, 6), 3402: (6, 7, 9, 9), 3456: (6, 6, 6, 16),
    3520: (11, 10, 8, 4), 3584: (2, 7, 16, 16), 3600: (10, 10, 9, 4), 3640: (13, 10, 7, 4),
    3696: (11, 8, 7, 6), 3744: (3, 6, 13, 16), 3780: (6, 7, 9, 10), 3840: (3, 5, 16, 16),
    3850: (5, 7, 10, 11), 3872: (11, 11, 8, 4), 3888: (9, 9, 8, 6), 3920: (10, 8, 7, 7),
    3960: (11, 10, 9, 4), 4032: (9, 8, 8, 7), 4095: (5, 7, 9, 13),
}

# --all-variants lists every candidate thread count of every length (a tuning build)
ALL_VARIANTS = "--all-variants" in sys.argv[1:]
# --only=<p>,<q>,...: with --all-variants, only lengths divisible by one of these get variants
ONLY = [int(v) for a in sys.argv[1:] if a.startswith("--only=") for v in a[7:].split(",")]

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


def lds_bytes(n, elem_bytes):
    pitch = (n + ((n - 1) >> 4) + 1) | 1
    return pitch * elem_bytes


def best_schedule(n, max_threads=512):
    best = None
    for npass in range(1, 5):
        for combo in itertools.combinations_with_replacement(RADICES, npass):
            prod = 1
            for r in combo:
                prod *= r
            if prod != n:
                continue
            t = tpt(n, combo)
            if t > max_threads:
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
    for p in (2, 3, 5, 7, 11, 13):
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
    for n in WIDE_LENGTHS:
        s = TUNED_SCHEDULE.get(n) or best_schedule(n, 1024)
        rows.append((n, s, 0))
    out = sys.stdout
    out.write("// fast_schedules.h -- generated by gen_fast_schedules.py, do not edit.\n")
    out.write("// FAST_SCHED(slice, all_modes, N, R0, R1, R2, R3, TPTF, TPTD, DBL): length N runs the passes R0..R3\n")
    out.write("// (1 = unused) with TPTF / TPTD threads per transform in single / double precision (0 = the\n")
    out.write("// fewest the register budget allows); DBL = 0: no double-precision kernel (it would not fit);\n")
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
        if ALL_VARIANTS and (not ONLY or any(n % q == 0 for q in ONLY)):
            variants = [(sc, t, t) for sc, t in tuning_variants(n)]
        else:
            tf, td = TUNED_TPT.get(n, (0, 0))
            variants = [(s, tf, td)]
        for sc, tf, td in variants:
            r = list(sc) + [1] * (4 - len(sc))
            dbl = 1 if (max(td, tpt(n, sc)) <= 512 and lds_bytes(n, 16) <= LDS_BYTES) else 0
            out.write("FAST_SCHED(%d, %d, %d, %d, %d, %d, %d, %d, %d, %d)\n"
                      % (slice_of[n], full, n, r[0], r[1], r[2], r[3], tf, td, dbl))
    sys.stderr.write("%d lengths\n" % len(rows))


if __name__ == "__main__":
    main()
