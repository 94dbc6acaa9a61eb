"""Build step: puts the 8-byte instructions of gfx950 device assembly on 8-byte boundaries.

A wave that has a SIMD to itself (the regime of the small-batch sweeps: one wave per SIMD) issues an 8-byte
instruction that starts at an offset of 4 modulo 8 about 15 % slower than an aligned one (measured: 2.16 against
1.89 ns per v_fma_f64); 4-byte instructions do not care.  The compiler lays instructions out without regard to this.
This pass walks every function of an assembly file and, by dynamic programming over the layout, chooses for each
4-byte VALU instruction whether to keep it or to emit it in its equivalent 8-byte encoding (`_e32` -> `_e64`: same
operation, same operands, no extra issue slot), and whether to pad with an `s_nop` (one issue slot, only ahead of long
runs), so that as few 8-byte instructions as possible start misaligned.  The arithmetic is untouched.

usage: align_pass.py in.s out.s     (in.s: `hipcc --cuda-device-only -S`; the Makefile assembles and embeds out.s)
"""
import os
import re
import subprocess
import sys
import tempfile

LLVM = os.environ.get("LLVM_BIN", "/opt/rocm/lib/llvm/bin")
ARCH = os.environ.get("ARCH", "gfx950")
# an s_nop costs a whole issue slot, a misaligned instruction about a seventh of one
NOP_COST = float(os.environ.get("ALIGN_NOP_COST", "7"))


def assemble(path_s, path_o):
    subprocess.check_call([LLVM + "/clang", "-target", "amdgcn-amd-amdhsa", "-mcpu=" + ARCH, "-c", path_s, "-o", path_o])


def layout(path_o):
    """[(function, [(mnemonic, address, size), ...])] in layout order, from the disassembly of an object file"""
    out = subprocess.check_output([LLVM + "/llvm-objdump", "-d", path_o], text=True)
    funcs, cur = [], None
    for line in out.split("\n"):
        m = re.match(r"^[0-9a-f]+ <(.+)>:$", line)
        if m:
            cur = (m.group(1), [])
            funcs.append(cur)
            continue
        m = re.match(r"^\s+(\S+).*// ([0-9A-F]+): ((?:[0-9A-F]{8} ?)+)", line)
        if m and cur is not None:
            cur[1].append((m.group(1), int(m.group(2), 16), 4 * len(m.group(3).split())))
    return funcs


def instruction_lines(src):
    """{function: [index of each instruction line, in order]}"""
    funcs, cur = {}, None
    for i, line in enumerate(src):
        s = line.strip()
        m = re.match(r"^([A-Za-z_][\w$.]*):", line)
        if m and not s.startswith(".L"):
            cur = funcs.setdefault(m.group(1), [])
            continue
        if cur is None or not s or s[0] in ";." or re.match(r"^[\w$.]+:", s):
            continue
        cur.append(i)
    return funcs


def plan(ins, text, start_parity):
    """Per instruction 'keep', 'wide' (re-encode in 8 bytes) or 'nop' (pad ahead of it); parity 1 = offset 4 mod 8."""
    n = len(ins)
    cost = [[0.0, 0.0] for _ in range(n + 1)]
    act = [[None, None] for _ in range(n)]
    for k in range(n - 1, -1, -1):
        mn, _, size = ins[k]
        widenable = (size == 4 and mn.endswith("_e32") and mn in text[k]
                     and not mn.startswith(("v_readfirstlane", "v_nop", "v_swap")))
        words = size // 4
        for p in (0, 1):
            if size >= 8:
                best, how = p + cost[k + 1][(p + words) % 2], "keep"
                c = NOP_COST + (1 - p) + cost[k + 1][(p + 1 + words) % 2]
                if c < best:
                    best, how = c, "nop"
            else:
                best, how = cost[k + 1][1 - p], "keep"
                if widenable:
                    c = p + cost[k + 1][p]
                    if c < best:
                        best, how = c, "wide"
            cost[k][p], act[k][p] = best, how
    out, p = [], start_parity
    for k in range(n):
        how = act[k][p]
        out.append(how)
        words = ins[k][2] // 4
        p = p if how == "wide" else (p + words + (1 if how == "nop" else 0)) % 2
    return out


def main():
    src = open(sys.argv[1]).read().split("\n")
    tmp = tempfile.mkdtemp()
    try:
        assemble(sys.argv[1], tmp + "/a.o")
        lines = instruction_lines(src)
        before = wide = nops = 0
        for name, ins in layout(tmp + "/a.o"):
            idx = lines.get(name)
            if not ins or idx is None or len(idx) != len(ins):
                continue        # cannot be matched line by line: left as it is
            before += sum(1 for (_, addr, size) in ins if size >= 8 and addr % 8 == 4)
            for k, how in enumerate(plan(ins, [src[i] for i in idx], (ins[0][1] // 4) % 2)):
                if how == "wide":
                    mn = ins[k][0]
                    src[idx[k]] = src[idx[k]].replace(mn, mn[:-4] + "_e64", 1)
                    wide += 1
                elif how == "nop":
                    src[idx[k]] = "\ts_nop 0\n" + src[idx[k]]
                    nops += 1
        open(sys.argv[2], "w").write("\n".join(src))
        assemble(sys.argv[2], tmp + "/b.o")
        left = sum(1 for _, ins in layout(tmp + "/b.o") for (_, addr, size) in ins if size >= 8 and addr % 8 == 4)
        print("align_pass %s: 8-byte instructions at offset 4 mod 8: %d -> %d (%d re-encoded, %d s_nop)"
              % (os.path.basename(sys.argv[1]), before, left, wide, nops), file=sys.stderr)
    finally:
        for f in os.listdir(tmp):
            os.remove(os.path.join(tmp, f))
        os.rmdir(tmp)


if __name__ == "__main__":
    main()
