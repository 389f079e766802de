"""Generates walk_asm.inc: the hand-scheduled stage walk of the plain simulator.

    python mms_amd/csrc/gen_walk_asm.py        # rewrites walk_asm.inc next to this file

One inline-asm block per request does, for the lanes of a wavefront:

  fetch   c[k] = clk[slot0 + k]            for k <= walk      (ds_read_b64)
  chain   t = max(t, c[k]) + lat[k]; c[k] = t                 (v_max_f64, v_add_f64)
          finish = t + overhead at the lane's last level
  decide  latency = finish - arrival; accept = latency <= slo
  commit  clk[slot0 + k] = c[k]            for accepted lanes, k <= walk

which is the loop body of the reference's simulate_requests_mixed
(alpa_serve/simulator/controller.py:605-619).  `walk` is a lane's stage count
minus one, or -1 for lanes that do not dispatch.  Per level EXEC is narrowed
with one v_cmpx (lanes leave in order of depth, so narrowing is monotone) and
restored once per phase; a wave-uniform exit is tested only at depths 1, 2, 4,
8 and 16.  Temporaries live in fixed registers that are declared clobbered.

Two flavours: "U" (one latency per (model, config): operand lc) and "N"
(per-stage latencies read from the LDS table at byte address lb).

The "P" variants are for batches whose pipeline depths are all powers of two
(the usual case: group sizes and their inter-op splits are 1, 2, 4, 8, 16).
Lanes can then only leave at depths 1, 2, 4, 8, so EXEC is narrowed there and
nowhere else, clock slots move two at a time (ds_read2st64_b64 /
ds_write2st64_b64: the 512-byte slot pitch is exactly the st64 stride), and the
finish time is formed at the four exits instead of tracking t per level.
"""
import os

C0 = 200      # c[k] = v[C0+2k : C0+2k+1]
L0 = 234      # l[k] = v[L0+k]                     (N flavour)
TMP = 232     # v[TMP:TMP+1] widened latency       (N flavour)
EXITS = (1, 2, 4, 8, 16)


def creg(k):
    return f"v[{C0 + 2 * k}:{C0 + 2 * k + 1}]"


def narrow(k):
    return f"v_cmpx_le_i32_e32 vcc, {k}, %[walk]"


def body(levels, flavour):
    a = []
    a.append("s_mov_b64 %[sv], exec")
    a.append("v_mov_b32_e32 %[acc], 0")
    # ---- fetch
    a.append(narrow(0))
    a.append("s_cbranch_execz .Lmmsim_end_%=")
    for k in range(levels):
        if k > 0:
            a.append(narrow(k))
            if k in EXITS:
                a.append("s_cbranch_execz .Lmmsim_fetched_%=")
        a.append(f"ds_read_b64 {creg(k)}, %[cb]" + (f" offset:{512 * k}" if k else ""))
        if flavour == "N":
            a.append(f"ds_read_b32 v{L0 + k}, %[lb]" + (f" offset:{4 * k}" if k else ""))
    a.append(".Lmmsim_fetched_%=:")
    a.append("s_mov_b64 exec, %[sv]")
    # ---- chain
    a.append(narrow(0))
    a.append("s_waitcnt lgkmcnt(0)")
    for k in range(levels):
        if k > 0:
            a.append(narrow(k))
            if k in EXITS:
                a.append("s_cbranch_execz .Lmmsim_chained_%=")
        prev = "%[ts]" if k == 0 else creg(k - 1)
        a.append(f"v_max_f64 {creg(k)}, {prev}, {creg(k)}")
        if flavour == "N":
            a.append(f"v_cvt_f64_f32_e32 v[{TMP}:{TMP + 1}], v{L0 + k}")
            a.append(f"v_add_f64 {creg(k)}, {creg(k)}, v[{TMP}:{TMP + 1}]")
        else:
            a.append(f"v_add_f64 {creg(k)}, {creg(k)}, %[lc]")
        a.append(f"v_add_f64 %[fin], {creg(k)}, %[oh]")   # off the chain; the lane's last level wins
    a.append(".Lmmsim_chained_%=:")
    a.append("s_mov_b64 exec, %[sv]")
    # ---- decide
    a.append(narrow(0))
    a.append("v_add_f64 %[lat], %[fin], -%[ts]")
    a.append("v_cmpx_le_f64_e32 vcc, %[lat], %[slo]")
    a.append("s_cbranch_execz .Lmmsim_end_%=")
    a.append("v_mov_b32_e32 %[acc], 1")
    a.append("v_add_u32_e32 %[ng], 1, %[ng]")
    a.append("v_add_f64 %[ls], %[ls], %[lat]")
    # ---- commit
    for k in range(levels):
        if k > 0:
            a.append(narrow(k))
            if k in EXITS:
                a.append("s_cbranch_execz .Lmmsim_end_%=")
        a.append(f"ds_write_b64 %[cb], {creg(k)}" + (f" offset:{512 * k}" if k else ""))
    a.append(".Lmmsim_end_%=:")
    a.append("s_mov_b64 exec, %[sv]")
    return a


def pairs(lo, hi):
    """LDS moves for levels lo..hi-1 (lo even or hi-lo == 1): (mnemonic suffix, first level)."""
    out = []
    k = lo
    while k < hi:
        if k % 2 == 0 and k + 1 < hi:
            out.append((2, k))
            k += 2
        else:
            out.append((1, k))
            k += 1
    return out


def body_pow2(levels, flavour):
    # depth blocks [0,1) [1,2) [2,4) [4,8) [8,16): lanes inside a block all stay to its end
    blocks = [(0, 1)] + [(e, min(2 * e, levels)) for e in EXITS if e < levels]
    a = []
    a.append("s_mov_b64 %[sv], exec")
    a.append("v_mov_b32_e32 %[acc], 0")
    # ---- fetch
    for lo, hi in blocks:
        a.append(narrow(lo))
        a.append("s_cbranch_execz " + (".Lmmsim_end_%=" if lo == 0 else ".Lmmsim_fetched_%="))
        for n, k in pairs(lo, hi):
            if n == 2:
                a.append(f"ds_read2st64_b64 v[{C0 + 2 * k}:{C0 + 2 * k + 3}], %[cb] offset0:{k} offset1:{k + 1}")
            else:
                a.append(f"ds_read_b64 {creg(k)}, %[cb]" + (f" offset:{512 * k}" if k else ""))
        if flavour == "N":
            for k in range(lo, hi):
                a.append(f"ds_read_b32 v{L0 + k}, %[lb]" + (f" offset:{4 * k}" if k else ""))
    a.append(".Lmmsim_fetched_%=:")
    a.append("s_mov_b64 exec, %[sv]")
    # ---- chain
    for lo, hi in blocks:
        a.append(narrow(lo))
        if lo == 0:
            a.append("s_waitcnt lgkmcnt(0)")
        else:
            a.append("s_cbranch_execz .Lmmsim_chained_%=")
        for k in range(lo, hi):
            prev = "%[ts]" if k == 0 else creg(k - 1)
            a.append(f"v_max_f64 {creg(k)}, {prev}, {creg(k)}")
            if flavour == "N":
                a.append(f"v_cvt_f64_f32_e32 v[{TMP}:{TMP + 1}], v{L0 + k}")
                a.append(f"v_add_f64 {creg(k)}, {creg(k)}, v[{TMP}:{TMP + 1}]")
            else:
                a.append(f"v_add_f64 {creg(k)}, {creg(k)}, %[lc]")
        a.append(f"v_add_f64 %[fin], {creg(hi - 1)}, %[oh]")
    a.append(".Lmmsim_chained_%=:")
    a.append("s_mov_b64 exec, %[sv]")
    # ---- decide
    a.append(narrow(0))
    a.append("v_add_f64 %[lat], %[fin], -%[ts]")
    a.append("v_cmpx_le_f64_e32 vcc, %[lat], %[slo]")
    a.append("s_cbranch_execz .Lmmsim_end_%=")
    a.append("v_mov_b32_e32 %[acc], 1")
    a.append("v_add_u32_e32 %[ng], 1, %[ng]")
    a.append("v_add_f64 %[ls], %[ls], %[lat]")
    # ---- commit
    for lo, hi in blocks:
        if lo > 0:
            a.append(narrow(lo))
            a.append("s_cbranch_execz .Lmmsim_end_%=")
        for n, k in pairs(lo, hi):
            if n == 2:
                a.append(f"ds_write2st64_b64 %[cb], {creg(k)}, {creg(k + 1)} offset0:{k} offset1:{k + 1}")
            else:
                a.append(f"ds_write_b64 %[cb], {creg(k)}" + (f" offset:{512 * k}" if k else ""))
    a.append(".Lmmsim_end_%=:")
    a.append("s_mov_b64 exec, %[sv]")
    return a


def clobbers(levels, flavour):
    regs = [f"v{C0 + i}" for i in range(2 * levels)]
    if flavour == "N":
        regs += [f"v{TMP}", f"v{TMP + 1}"] + [f"v{L0 + k}" for k in range(levels)]
    return regs


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    out = ["// GENERATED by gen_walk_asm.py -- do not edit by hand.",
           "// Stage walk of the plain simulator as one inline-asm block per request.", ""]
    for levels in (4, 16):
        for flavour in ("U", "N", "PU", "PN"):
            name = f"MMSIM_WALK_{flavour}{levels}"
            lines = body_pow2(levels, flavour[1]) if flavour[0] == "P" else body(levels, flavour)
            flavour = flavour[-1]
            out.append(f"#define {name}_TEXT \\")
            out.extend(f'    "{l}\\n" \\' for l in lines[:-1])
            out.append(f'    "{lines[-1]}\\n"')
            regs = clobbers(levels, flavour)
            out.append(f"#define {name}_CLOBBERS " + ", ".join(f'"{r}"' for r in regs))
            out.append("")
    with open(os.path.join(here, "walk_asm.inc"), "w") as f:
        f.write("\n".join(out))
    print("wrote walk_asm.inc")


if __name__ == "__main__":
    main()
