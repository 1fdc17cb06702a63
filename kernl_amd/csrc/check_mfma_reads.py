"""Checks device assembly listings (hipcc -S --cuda-device-only) for reads of matrix-instruction results that come too
early.  The wide linear kernels issue their MFMAs from inline assembly (common.h, mfma16_inplace), so the compiler
inserts none of the wait states a read of the result needs (11 after an 8-pass `v_mfma_f32_16x16x32`): nothing but the
kernel's own `mfma16_inplace_results_landed` keeps the epilogue's first `v_accvgpr_read` away from the last MFMA.

The check follows the program TEXT, not the control flow: after every `v_mfma` it counts instructions up to the next
`v_accvgpr_read` and reports a kernel where fewer than MIN_DISTANCE lie between them without an `s_nop 15`.  That is
conservative for fall-through code, which is where an epilogue follows its main loop.

usage: check_mfma_reads.py listing.s [...]      exit status 1 when a kernel is reported"""
import re
import sys

MIN_DISTANCE = 12


def kernels(lines):
    starts = [i for i, l in enumerate(lines) if re.match(r"^_ZN\S*:\s", l)]
    for n, s in enumerate(starts):
        yield lines[s].split(":")[0], lines[s + 1 : starts[n + 1] if n + 1 < len(starts) else len(lines)]


def early_reads(body):
    """Returns (line offset, distance) of the first accumulator read that follows an MFMA too closely, or None."""
    since, guarded, seen_mfma = 0, False, False
    for i, line in enumerate(body):
        text = line.strip()
        if not text or text[0] in ";." or text.endswith(":"):
            continue
        if text.startswith("v_mfma"):
            seen_mfma, since, guarded = True, 0, False
            continue
        if text.startswith("s_nop 15"):
            guarded = True
        if text.startswith("v_accvgpr_read") and seen_mfma and not guarded and since < MIN_DISTANCE:
            return i, since
        since += 1
    return None


def main(paths):
    reported = checked = 0
    for path in paths:
        with open(path) as f:
            lines = f.read().split("\n")
        for name, body in kernels(lines):
            if not any(l.lstrip().startswith("v_mfma") for l in body):
                continue
            checked += 1
            hit = early_reads(body)
            if hit is not None:
                reported += 1
                print(f"{path}: {name}: v_accvgpr_read {hit[1]} instructions after an MFMA (listing line +{hit[0]})")
    print(f"{checked} kernels with matrix instructions checked, {reported} reported")
    return 1 if reported or not checked else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
