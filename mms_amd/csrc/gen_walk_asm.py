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
(the usual case: group sizes and their inter-op splits are 1, 2, 4, 8, 16);
see body_pow2_straight.
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


def body(levels, flavour, lean=False):
    a = []
    a.append("s_mov_b64 %[sv], exec")
    a.append("s_mov_b64 %[am], 0")
    if not lean:
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
    a.append("s_mov_b64 %[am], exec")
    a.append("s_cbranch_execz .Lmmsim_end_%=")
    if not lean:
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


FSEL = 252    # v[FSEL:FSEL+1]: the clock of the lane's own last stage


def body_pow2_straight(levels, flavour, lean=False):
    """"P" walks: depths all powers of two.

    EXEC is written seven times at most instead of once per phase and exit: which lanes reach depth
    2, 4, 8, 16 is kept as four SGPR masks; the code is straight-line per wave depth D (the deepest
    walking lane, tested deepest first: deep walks are the common and the expensive ones), every
    walking lane fetches and chains D levels (levels past a lane's own depth read clocks and latencies
    that are not its group's and compute values nobody uses), the clock of the lane's own last stage
    is selected with the masks, one add gives its finish time, and only the commit narrows EXEC.  LDS
    reads are waited for one by one, so the chain starts when the first arrives; the selects sit in the
    issue slots the dependent max/add chain leaves empty.

    lean: the variant for callers that only need goodput and latency sums (no per-lane accept flag, no
    finish time); %[am] always receives the mask of accepting lanes.
    """
    depths = [d for d in (1, 2, 4, 8, 16) if d <= levels]
    masks = {1: "%[m1]", 2: "%[m2]", 4: "%[m4]", 8: "%[m8]"}     # lanes with depth > key
    csel = f"v[{FSEL}:{FSEL + 1}]"
    a = []
    a.append("s_mov_b64 %[sv], exec")
    a.append("s_mov_b64 %[am], 0")
    if not lean:
        a.append("v_mov_b32_e32 %[acc], 0")
    a.append(narrow(0))
    a.append("s_cbranch_execz .Lmmsim_end_%=")
    for e in depths[:-1]:
        a.append(f"v_cmp_le_i32_e64 {masks[e]}, {e}, %[walk]")
    a.append(f"ds_read_b64 {creg(0)}, %[cb]")
    if flavour == "N":
        a.append(f"ds_read_b32 v{L0}, %[lb]")
    for e in reversed(depths[:-1]):             # the wave's depth is 2e for the largest e somebody goes beyond
        a.append(f"s_cmp_lg_u64 {masks[e]}, 0")
        a.append(f"s_cbranch_scc1 .Lmmsim_d{2 * e}_%=")
    for D in depths:                            # shallowest first: depth 1 falls through from the dispatch
        a.append(f".Lmmsim_d{D}_%=:")
        # reads in issue order, each with the levels it brings (clock k: ("c", k), latency k: ("l", k))
        issued = [[("c", 0)]] + ([[("l", 0)]] if flavour == "N" else [])
        for n, k in (pairs(1, D) if D > 1 else []):
            if n == 2:
                a.append(f"ds_read2st64_b64 v[{C0 + 2 * k}:{C0 + 2 * k + 3}], %[cb] offset0:{k} offset1:{k + 1}")
            else:
                a.append(f"ds_read_b64 {creg(k)}, %[cb] offset:{512 * k}")
            issued.append([("c", kk) for kk in range(k, k + n)])
            if flavour == "N":
                for kk in range(k, k + n):
                    a.append(f"ds_read_b32 v{L0 + kk}, %[lb] offset:{4 * kk}")
                    issued.append([("l", kk)])
        # reads return in order: an item is there when at most (reads issued after it) are outstanding
        # (one latency per (model, config): the reads after the first are waited for two at a time -- a wait is an
        # instruction like any other, and with two wavefronts on a SIMD the walk is bound by what it issues)
        arrive = {}
        for i, items in enumerate(issued):
            upto = i if flavour == "N" or i == 0 else min(len(issued) - 1, i + i % 2)
            for it in items:
                arrive[it] = len(issued) - 1 - upto
        fill = []                               # independent instructions to drop into the chain's gaps
        waited = 99
        for k in range(D):
            need = arrive[("c", k)] if flavour == "U" else min(arrive[("c", k)], arrive[("l", k)])
            need = min(need, 15)                # the counter field has four bits; waiting for fewer is only stricter
            if need < waited:
                a.append(f"s_waitcnt lgkmcnt({need})")
                waited = need
            prev = "%[ts]" if k == 0 else creg(k - 1)
            a.append(f"v_max_f64 {creg(k)}, {prev}, {creg(k)}")
            if flavour == "N":
                a.append(f"v_cvt_f64_f32_e32 v[{TMP}:{TMP + 1}], v{L0 + k}")
            elif fill:
                a.append(fill.pop(0))
            a.append(f"v_add_f64 {creg(k)}, {creg(k)}, " + (f"v[{TMP}:{TMP + 1}]" if flavour == "N" else "%[lc]"))
            if fill:
                a.append(fill.pop(0))
            if k + 1 in depths and k + 1 > 1:   # a lane of depth k+1 ends here: its last-stage clock is c[k]
                i = depths.index(k + 1)
                m = masks[depths[i - 1]]
                src = creg(0) if i == 1 else csel        # depth-1 lanes end at c[0]
                lo, hi = (C0, C0 + 1) if i == 1 else (FSEL, FSEL + 1)
                fill.append(f"v_cndmask_b32_e64 v{FSEL}, v{lo}, v{C0 + 2 * k}, {m}")
                fill.append(f"v_cndmask_b32_e64 v{FSEL + 1}, v{hi}, v{C0 + 2 * k + 1}, {m}")
        a.extend(fill)
        last = creg(0) if D == 1 else csel
        a.append(f"v_add_f64 %[fin], {last}, %[oh]")      # :610
        a.append("v_add_f64 %[lat], %[fin], -%[ts]")
        if D != depths[-1]:
            a.append("s_branch .Lmmsim_decide_%=")
    # ---- decide
    a.append(".Lmmsim_decide_%=:")
    a.append("v_cmpx_le_f64_e32 vcc, %[lat], %[slo]")
    a.append("s_mov_b64 %[am], exec")
    a.append("s_cbranch_execz .Lmmsim_end_%=")
    if not lean:
        a.append("v_mov_b32_e32 %[acc], 1")
    a.append("v_add_u32_e32 %[ng], 1, %[ng]")
    a.append("v_add_f64 %[ls], %[ls], %[lat]")
    # ---- commit: accepted lanes, each its own depth
    a.append(f"ds_write_b64 %[cb], {creg(0)}")
    for e in depths[:-1]:
        a.append(f"s_and_b64 exec, exec, {masks[e]}")
        a.append("s_cbranch_scc0 .Lmmsim_end_%=")
        for n, k in pairs(e, 2 * e):
            if n == 2:
                a.append(f"ds_write2st64_b64 %[cb], {creg(k)}, {creg(k + 1)} offset0:{k} offset1:{k + 1}")
            else:
                a.append(f"ds_write_b64 %[cb], {creg(k)} offset:{512 * k}")
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
            for lean in (False, True):
                name = f"MMSIM_WALK_{flavour}{levels}" + ("_LEAN" if lean else "")
                straight = flavour[0] == "P"
                fl = flavour[-1]
                lines = body_pow2_straight(levels, fl, lean) if straight else body(levels, fl, lean)
                out.append(f"#define {name}_TEXT \\")
                out.extend(f'    "{l}\\n" \\' for l in lines[:-1])
                out.append(f'    "{lines[-1]}\\n"')
                regs = clobbers(levels, fl)
                if straight:
                    regs += [f"v{FSEL}", f"v{FSEL + 1}"]
                out.append(f"#define {name}_CLOBBERS " + ", ".join(f'"{r}"' for r in regs))
                out.append("")
    with open(os.path.join(here, "walk_asm.inc"), "w") as f:
        f.write("\n".join(out))
    print("wrote walk_asm.inc")


if __name__ == "__main__":
    main()
