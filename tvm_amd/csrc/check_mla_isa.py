"""Build step for kernels_mla.hip: checks in the generated gfx950 assembly what the source cannot
guarantee on its own.

The MLA kernel keeps O in the accumulation registers a0..a255 and reaches them by number from
inline assembly, so the compiler must never place a value of its own there (it may, for values
that only pass through loads, stores and copies, once the ordinary registers run out), and it does
not see the global->LDS copy inside the assembly, so it cannot insert the wait states that the
hardware wants between a vector instruction that writes a scalar register (a lane read that
restores a spilled scalar) and a memory instruction that uses this register as its base.

usage: check_mla_isa.py <assembly file>; exit status 1 and a message if either rule is broken."""
import re
import sys


def instructions(text):
    """(line number, text, inside inline assembly) of every instruction."""
    inside = False
    for no, line in enumerate(text.split("\n"), 1):
        t = line.strip()
        if t.startswith(";;#ASMSTART"):
            inside = True
        elif t.startswith(";;#ASMEND"):
            inside = False
        elif t and not t.startswith(";") and not t.startswith(".") and not t.endswith(":"):
            yield no, t.split(";")[0].strip(), inside


def main(path):
    ins = list(instructions(open(path).read()))
    errors = []
    for no, t, inside in ins:
        if not inside and re.search(r"\ba(\d+|\[\d)", t):
            errors.append(f"line {no}: compiler-generated instruction uses an accumulation register: {t}")
    for k, (no, t, inside) in enumerate(ins):
        m = re.match(r"global_load_lds_dwordx4 v\d+, s\[(\d+):(\d+)\]", t)
        if not m:
            continue
        base = {int(m.group(1)), int(m.group(2))}
        states = 0
        for no2, t2, _ in reversed(ins[max(0, k - 8):k]):
            w = re.match(r"v_read(first)?lane_b32 s(\d+),", t2)
            if w and int(w.group(2)) in base and states < 5:
                errors.append(f"line {no}: {t} uses s{w.group(2)} {states} wait states after line {no2}: {t2}")
            n = re.match(r"s_nop (\d+)", t2)
            states += int(n.group(1)) + 1 if n else 1
    for e in errors[:20]:
        print("check_mla_isa:", e, file=sys.stderr)
    return 1 if errors else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1]))
