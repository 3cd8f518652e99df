#!/usr/bin/env python3
"""Writes the hand-scheduled K loop of the 4-wave 256x256 tile kernels (gemm_w4.h) as inline-assembly text.

    python3 gen_w4.py fp8 > w4_kloop_fp8.inc        (also: e5m2, e4e5, e5e4, fp4, bf16, f16, i8)
    python3 gen_w4.py clobbers fp8 > w4_clobbers_fp8.inc
    python3 gen_w4.py check                          (walks every kind through the wait-count checker)

One workgroup = 4 waves (one per SIMD), wave (wm, wn) owns the 128x128 quarter of a 256x256 output
tile: 8x8 MFMA tiles of 16x16, i.e. 256 accumulator registers a[0:255]; acc(i, j) of A row block i and
B row block j sits in a[(8i+j)*4 .. +3].  A K step is 128 bytes of every operand row (128 FP8 values,
256 FP4 values or 64 16-bit values); LDS holds two stages of 64 KB: stage s at s*65536, A rows at +0,
B rows at +32768, row r at r*128 with its eight 16-byte chunks XOR-swizzled (the layout the 8-wave
kernels use).  FP4 adds two 8 KB buffers of E8M0 scales behind the stages (16 scale bytes per row =
two K steps).

The text is the code of ONE asm statement that runs the whole K loop of one output tile (at least four
K steps, an even number):

  entry      (first tile of the workgroup only) copies of K steps 0 and 1 and of scale group 0
  per K step eight row blocks of MFMAs (row block i multiplies A fragment i with the eight B fragments);
             A fragments go through four buffers, the B fragments of the next step sit in the other of
             two register sets.  Two sync points (wait + s_barrier) per step, each followed by copies of
             step +2 into LDS that every wave has just declared free:
               X, in row block 1: this step's B fragments and A fragments 0..3 are in registers -> the
                  B half of the stage and the A rows of row blocks 0..3 ("A lo") take step +2; it also
                  publishes "A hi" (row blocks 4..7) of THIS step, which is read from here on;
               Y, in row block 5: A fragments 4..7 are in registers -> "A hi" takes step +2; it
                  publishes B and "A lo" of the NEXT step for the reads that follow.
             Every copy is waited for one and a half K steps after it was issued and two to three
             bursts overlap in time (one burst per step that must land within one step leaves the
             L2 -> LDS path idle for the latency of its first byte and then stalls the MFMAs).
  first two  the MFMAs of step 0 start from zero (no clearing pass).  When the caller says so (%[fe]) the
  K steps    accumulators still hold the PREVIOUS tile's sums: each row block is then read out, scaled,
             rounded to bf16 and stored just before step 0 overwrites it, between the MFMAs of the row
             block before -- the epilogue costs no MFMA-idle time and its stores are spread over a K step.
             Step 1 loads this tile's own epilogue scales (FP8) into registers that the caller carries
             to the next call.
  last two   the copies go to the NEXT tile's first two K steps (the caller passes the next tile's
  K steps    addresses, or the same tile's again when there is none), so the copy pipeline never drains
             between tiles; no fragments are prefetched across the tile boundary.

vmcnt counts vector-memory operations in issue order, loads and stores alike, so every wait names how
many YOUNGER operations may still be in flight.  Those numbers depend on what ran before (the entry's
copies, a previous tile's epilogue stores issued by compiled code, the fused epilogue's own stores);
`check` replays the instruction stream of every such history and proves each wait at least as strict
as needed.

Register map (VGPR):  0..127   B fragment sets 0/1 (8 fragments x 8 registers each)
                      128..159 A fragment buffers 0..3
                      160..191 FP4: E8M0 scale registers (set p: A rows 160+16p+i, B rows 168+16p+j);
                               FP8: epilogue column scales sb (in/out)
                      192..207 in: byte offsets of this tile's copies (A 192+i, B 200+i, i = copy instruction)
                      208..223 in: the same for the next tile
                      224..231 in: fragment read addresses (A lo, A hi, B lo, B hi) for stage 0, then stage 1
                      FP4:  232..237 in: scale read addresses (A, B), scale copy offsets (A, B) now and next;
                            238 in: C offset of this lane; 240, 241 scale read addresses of the current buffer
                      else: 240 in: C offset of this lane; FP8: 241 in: lane * 4, 242 in / 243 in: LDS
                            addresses this lane reads its row / column scales from
                      The fused epilogue works in B fragment set 1 (64..127), which is free from the end of
                      the previous tile until the second half of step 0: column scales 64..95, row scales
                      96..103, scratch 104..113.
SGPR 70..89 are scratch (copy cursors, loop counter, scale buffer toggle, flags, C row pointer).
"""
import os
import re
import sys

STAGE = 65536
BOFF = 32768
SC0 = 131072          # scale buffers behind the two stages
SCBUF = 8192
EPS = SC0 + 2 * SCBUF  # epilogue scales: 1 KB per wave
NST = 32              # stores per wave of an epilogue (256x256 16-bit values, 16 bytes per lane and store)

S_CA, S_CB, S_CSA, S_CSB, S_CNT, S_SCN, S_T, S_SCIN, S_AFTER, S_CROW, S_T2 = 70, 72, 74, 76, 78, 79, 80, 81, 82, 84, 86


class Op:
    """one instruction; vm: tag of the group of vector-memory operations it belongs to (None: not one)"""
    def __init__(self, text, vm=None):
        self.text, self.vm = text, vm


class WaitVm:
    """s_waitcnt vmcnt(n): everything up to and including group `awaits` must have completed.  vals maps
    a history ("a" first tile of the workgroup, "b" previous tile's epilogue = 32 compiled stores, "c" =
    unknown compiled stores, "d" fused epilogue, "s" steady state, "f" first even step after the first
    two) to n."""
    def __init__(self, awaits, vals):
        # vals: {history: n}, or a list of histories whose n the generator works out by replay (Gen.solve)
        if not isinstance(vals, dict):
            vals = {k: None for k in vals}
        self.awaits, self.vals = awaits, {k: (None if v is None else min(63, v)) for k, v in vals.items()}


F8_KINDS = ("fp8", "e5m2", "e4e5", "e5e4")


class Gen:
    def __init__(self, kind, lab=()):
        self.kind = kind                # "fp8" | "e5m2" | "e4e5" | "e5e4" | "fp4" | "bf16" | "f16" | "i8"
        # 8-bit floats: one MFMA of K = 128 per fragment pair; the kinds differ in its format fields (e4e5: A in e4m3, B in
        # e5m2; e5e4 the other way round)
        self.f8 = kind in F8_KINDS
        self.fp4 = kind == "fp4"        # (the only kind with E8M0 scale operands)
        self.scaled_epi = kind in F8_KINDS or kind == "i8"  # the fused epilogue multiplies by sa[m] * sb[n]
        self.int_acc = kind == "i8"      # int32 sums: converted to fp32 where they leave the accumulators
        self.nm = 8 if self.f8 else 16      # MFMAs per row block (FP8: one of K = 128 per fragment pair; others: two half-K ones)
        self.nsc = 4 if self.scaled_epi else 0    # copies of the tile's own epilogue scales (step 1)
        self.lbl = 0
        # how far (in MFMAs) into row blocks 1 and 5 the two sync points of a K step sit
        self.xoff = int(os.environ.get("W4GEN_XOFF", str(self.nm // 2)))
        self.yoff = int(os.environ.get("W4GEN_YOFF", str(self.nm // 2)))
        # measurement builds (W4GEN_LAB=nomfma,nodma,dmaonce,noread,nobar,novm,nolgk,m0nop,nostore): leave one kind of
        # instruction out (noscale: the MXFP4 kernel's scale copies and scale reads) to time the rest; results are then meaningless.  dmaonce = nodma except for the
        # first tile's entry copies, so that the LDS holds real operand data for the MFMAs to chew on.
        self.lab = set(lab)
        # earlyb: the B rows of fragments 0..3 (copied first) are published by the X of the step after the copy instead of
        # its Y, and the next step's B fragments 0..3 are read between X and Y (the LDS is idle there and the stretch
        # behind Y cannot take all the fragment reads); earlysc (MXFP4): the scale copy leads that group, so the next
        # step's scale reads move in front of Y in every step, not only in those that stay inside a scale group
        self.earlyb = os.environ.get("W4GEN_EARLYB", "1" if kind == "fp4" else "0") == "1"
        self.earlysc = os.environ.get("W4GEN_EARLYSC", "0") == "1"
        self.v_coff = 238 if self.fp4 else 240
        self.v_lane4, self.v_sa_rd, self.v_sb_rd = 241, 242, 243
        self.v_sb, self.v_sa, self.epi_tmp = 64, 96, 104

    # ---- register names ---------------------------------------------------------------------------
    @staticmethod
    def vB(p, j):
        return p * 64 + j * 8

    @staticmethod
    def vA(b):
        return 128 + (b % 4) * 8

    @staticmethod
    def scA(p, i):
        return 160 + p * 16 + i

    @staticmethod
    def scB(p, j):
        return 168 + p * 16 + j

    @staticmethod
    def fa(op, hi, stage):          # op: 0 = A, 1 = B
        return 224 + stage * 4 + op * 2 + hi

    # ---- building blocks --------------------------------------------------------------------------
    def frag_read(self, dst, op, stage, t):
        """both 16-byte halves of fragment t (16 rows x 128 bytes of K) of operand op"""
        return [Op(f"ds_read_b128 v[{dst}:{dst + 3}], v{self.fa(op, 0, stage)} offset:{t * 2048}"),
                Op(f"ds_read_b128 v[{dst + 4}:{dst + 7}], v{self.fa(op, 1, stage)} offset:{t * 2048}")]

    def scale_reads(self, p, half):
        """E8M0 bytes of one K step for all row blocks: two bytes (k slices 0, 1) per lane and row block"""
        r = []
        for i in range(8):
            r.append(Op(f"ds_read_u16 v{self.scA(p, i)}, v240 offset:{i * 256 + half * 8}"))
        for j in range(8):
            r.append(Op(f"ds_read_u16 v{self.scB(p, j)}, v241 offset:{j * 256 + half * 8}"))
        return r

    def dma(self, stage, nxt, tag):
        """the 16 LDS-direct copies of one K step (A then B), each as [m0 setup, wait state, load]"""
        ops = []
        base = 208 if nxt else 192
        for op, cur in ((0, S_CA), (1, S_CB)):
            for i in range(8):
                imm = stage * STAGE + op * BOFF + i * 4096
                ops.append([Op(f"s_add_u32 m0, %[wl], {imm}"), Op("s_nop 0"),
                            Op(f"global_load_lds_dwordx4 v{base + op * 8 + i}, s[{cur}:{cur + 1}]", tag)])
        return ops

    def dma_advance(self):
        return [Op(f"s_add_u32 s{S_CA}, s{S_CA}, 128"), Op(f"s_addc_u32 s{S_CA + 1}, s{S_CA + 1}, 0"),
                Op(f"s_add_u32 s{S_CB}, s{S_CB}, 128"), Op(f"s_addc_u32 s{S_CB + 1}, s{S_CB + 1}, 0")]

    def scale_dma(self, nxt, tag):
        """copy of one scale group (16 bytes per row, A rows then B rows) into the buffer s79 names, then toggle it"""
        va, vb = (236, 237) if nxt else (234, 235)
        return [[Op(f"s_add_u32 s{S_T}, %[wl], s{S_SCN}"), Op(f"s_add_u32 m0, s{S_T}, {SC0}"), Op("s_nop 0"),
                 Op(f"global_load_lds_dwordx4 v{va}, s[{S_CSA}:{S_CSA + 1}]", tag)],
                [Op(f"s_add_u32 m0, s{S_T}, {SC0 + 4096}"), Op("s_nop 0"),
                 Op(f"global_load_lds_dwordx4 v{vb}, s[{S_CSB}:{S_CSB + 1}]", tag),
                 Op(f"s_xor_b32 s{S_SCN}, s{S_SCN}, {SCBUF}"),
                 Op(f"s_add_u32 s{S_CSA}, s{S_CSA}, 16"), Op(f"s_addc_u32 s{S_CSA + 1}, s{S_CSA + 1}, 0"),
                 Op(f"s_add_u32 s{S_CSB}, s{S_CSB}, 16"), Op(f"s_addc_u32 s{S_CSB + 1}, s{S_CSB + 1}, 0")]]

    def mfma(self, p, i, slot, zero):
        """MFMA number `slot` of row block i: B fragment first (its rows become the output rows a lane
        holds).  zero: first K step of a tile, the sum starts from 0 instead of the accumulator."""
        if self.f8:
            j = slot
            acc = (i * 8 + j) * 4
            b, a = self.vB(p, j), self.vA(i)
            c = "0" if zero else f"a[{acc}:{acc + 3}]"
            # format fields: cbsz = the first source (the B fragment), blgp = the second (the A fragment); e4m3 is the default
            fmt = {"fp8": "", "e5m2": " cbsz:1 blgp:1", "e4e5": " cbsz:1", "e5e4": " blgp:1"}[self.kind]
            return Op(f"v_mfma_f32_16x16x128_f8f6f4 a[{acc}:{acc + 3}], v[{b}:{b + 7}], v[{a}:{a + 7}], {c}{fmt}")
        # two MFMAs per accumulator and K step, k slice outermost so that the same accumulator comes up
        # again only eight instructions later
        ks, j = slot // 8, slot % 8
        acc = (i * 8 + j) * 4
        b, a = self.vB(p, j) + 4 * ks, self.vA(i) + 4 * ks
        c = "0" if (zero and ks == 0) else f"a[{acc}:{acc + 3}]"
        if self.kind in ("bf16", "f16"):
            return Op(f"v_mfma_f32_16x16x32_{self.kind} a[{acc}:{acc + 3}], v[{b}:{b + 3}], v[{a}:{a + 3}], {c}")
        if self.kind == "i8":
            return Op(f"v_mfma_i32_16x16x64_i8 a[{acc}:{acc + 3}], v[{b}:{b + 3}], v[{a}:{a + 3}], {c}")
        return Op(f"v_mfma_scale_f32_16x16x128_f8f6f4 a[{acc}:{acc + 3}], v[{b}:{b + 3}], v[{a}:{a + 3}], {c}, "
                  f"v{self.scB(p, j)}, v{self.scA(p, i)} op_sel:[{ks},{ks},0] op_sel_hi:[0,0,0] cbsz:4 blgp:4")

    def epilogue_block(self, i, tag, f16=False):
        """The previous tile's row block i: for each of its four column groups read eight sums, scale
        (FP8: acc * (sa[m] * sb[n]), the order the compiled epilogues use), round to bf16 pairs, store 16
        bytes.  Returns the instructions in order; the row pointer s[84:85] moves on afterwards."""
        t = self.epi_tmp
        e = [t, t + 1, t + 2, t + 3]
        s, pk = t + 4, [t + 6, t + 7, t + 8, t + 9]     # (register tuples start at even registers)
        out = []
        for q in range(4):
            for h in range(2):
                base = (i * 8 + 2 * q + h) * 4
                for x in range(4):
                    out.append(Op(f"v_accvgpr_read_b32 v{e[x]}, a{base + x}"))
                if self.int_acc:
                    for x in range(4):
                        out.append(Op(f"v_cvt_f32_i32 v{e[x]}, v{e[x]}"))
                if self.scaled_epi:
                    for x in range(4):
                        out.append(Op(f"v_mul_f32 v{s}, v{self.v_sa + i}, v{self.v_sb + q * 8 + h * 4 + x}"))
                        out.append(Op(f"v_mul_f32 v{e[x]}, v{e[x]}, v{s}"))
                cvt = "v_cvt_pk_f16_f32" if f16 else "v_cvt_pk_bf16_f32"
                out.append(Op(f"{cvt} v{pk[2 * h]}, v{e[0]}, v{e[1]}"))
                out.append(Op(f"{cvt} v{pk[2 * h + 1]}, v{e[2]}, v{e[3]}"))
            out.append(Op(f"global_store_dwordx4 v{self.v_coff}, v[{pk[0]}:{pk[3]}], s[{S_CROW}:{S_CROW + 1}] offset:{q * 64}", tag))
        out.append(Op(f"s_add_u32 s{S_CROW}, s{S_CROW}, %[cstep]"))
        out.append(Op(f"s_addc_u32 s{S_CROW + 1}, s{S_CROW + 1}, 0"))
        return out

    def scale_loads(self, tag):
        """This tile's own epilogue scales (sa of the wave's 128 rows, sb of its 128 columns: 2 x 512 bytes)
        go to the wave's 1 KB of LDS behind the stages; the tile that runs the epilogue reads them there."""
        out = [Op(f"s_mov_b64 s[{S_T2}:{S_T2 + 1}], %[sap]")]
        for n, (base, half) in enumerate((("sap", 0), ("sap", 1), ("sbp", 0), ("sbp", 1))):
            if half == 0:
                out.append(Op(f"s_mov_b64 s[{S_T2}:{S_T2 + 1}], %[{base}]"))
            else:
                out += [Op(f"s_add_u32 s{S_T2}, s{S_T2}, 256"), Op(f"s_addc_u32 s{S_T2 + 1}, s{S_T2 + 1}, 0")]
            out += [Op(f"s_add_u32 m0, %[wl], {EPS + n * 256}"), Op("s_nop 0"),
                    Op(f"global_load_lds_dword v{self.v_lane4}, s[{S_T2}:{S_T2 + 1}]", tag)]
        return out[1:]

    def scale_reads_epi(self):
        """the previous tile's scales of this lane: rows 16 i + r, columns 32 q + 8 g + 0..7"""
        out = []
        for i in range(8):
            out.append(Op(f"ds_read_b32 v{self.v_sa + i}, v{self.v_sa_rd} offset:{i * 64}"))
        for q in range(4):
            for h in range(2):
                r = self.v_sb + q * 8 + h * 4
                out.append(Op(f"ds_read_b128 v[{r}:{r + 3}], v{self.v_sb_rd} offset:{q * 128 + h * 16}"))
        return out

    # ---- one K step -------------------------------------------------------------------------------
    def step(self, p, nxt, prefetch, flavor="steady", pending0=None):
        """K step in stage p (= B set p, scale set p).  nxt: the copies issued in this step read the
        next tile.  prefetch: request the following step's fragments.  flavor: "steady", "first0" (step 0
        of a tile), "first0_fe" (with the previous tile's epilogue fused in), "first1".  Group tags are
        relative to this step: ("XB", 0) / ("X", 0) / ("Y", 0) are issued, ("Y", -2) or ("XB", -1) and
        ("X", -1) awaited.  pending0: the LDS reads that may still be in flight when the step starts
        (oldest first, one set of destination registers each)."""
        nm = self.nm
        total = 8 * nm
        first0 = flavor in ("first0", "first0_fe", "first0_fe16")
        fe = flavor in ("first0_fe", "first0_fe16")
        eb = self.earlyb
        # early: the next step's B fragments 0..3 (and E8M0 scales) are read between X and Y instead of behind Y
        early = eb and prefetch and not fe
        q = p ^ 1
        out = [Op(f"; ---- K step, stage {p}, {flavor}{' (copies: next tile)' if nxt else ''}{'' if prefetch else ' (last of the tile)'}")]
        pre = [[] for _ in range(total)]      # in front of MFMA slot m
        post = [[] for _ in range(total)]     # behind it
        ops = self.dma(p, nxt, None)
        a_lo = [ops[i] for i in (0, 1, 4, 5)]                 # A rows of row blocks 0..3 (both wave rows)
        a_hi = [ops[i] for i in (2, 3, 6, 7)]
        b_lo = [ops[8 + i] for i in (0, 1, 4, 5)]             # B rows of fragments 0..3 (both wave columns)
        b_hi = [ops[8 + i] for i in (2, 3, 6, 7)]
        has_sc = self.fp4 and p == 0
        if eb:
            # what the next step's X waits for comes first
            sc_head = has_sc and self.earlysc
            sc = self.scale_dma(nxt, ("XB", 0) if sc_head else ("X", 0)) if has_sc else []
            for o in b_lo:
                o[-1].vm = ("XB", 0)
            for o in b_hi + a_lo:
                o[-1].vm = ("X", 0)
            xops = (sc if sc_head else []) + b_lo + b_hi + a_lo + ([] if sc_head else sc)
        else:
            sc = self.scale_dma(nxt, ("X", 0)) if has_sc else []
            for o in ops[8:] + a_lo:
                o[-1].vm = ("X", 0)
            xops = ops[8:] + a_lo + sc
        for o in a_hi:
            o[-1].vm = ("Y", 0)
        adv = self.dma_advance()
        adv_a, adv_b = adv[:2], adv[2:]
        nsc = self.nsc
        if fe:
            # fused epilogue: row block 0 in front of the first MFMA, the others spread over row blocks 0..4:
            # block k is done before slot 5 nm k / 7 <= nm k, where its accumulators are overwritten, and
            # everything is done before the fragments of step 1 arrive in the registers used here
            blocks = [self.epilogue_block(i, ("ST", 0), flavor == "first0_fe16") for i in range(8)]
            pre[0] += blocks[0]
            rest = [o for b in blocks[1:] for o in b]
            for n, o in enumerate(rest):
                post[n * 5 * nm // len(rest)].append(o)
        # row block 0
        if flavor == "first1" and nsc:
            pre[0] += self.scale_loads(("SC", 0))
        pre[0] += self.frag_read(self.vA(3), 0, p, 3)
        xs = nm + self.xoff
        tail0 = 5 * nm + self.yoff
        # X: history keys of the waits (the counts are worked out by replay, see solve)
        keys = {"steady": ["s"], "first0": ["a", "b", "c"], "first0_fe": ["d"], "first0_fe16": ["d"], "first1": ["a", "b", "c", "d"]}[flavor]
        keys_x = ["s", "f"] if (flavor == "steady" and p == 0 and nsc) else keys
        wx = WaitVm(("XB", -1) if early else ("Y", -2), keys_x)
        pre[xs] += [Op("s_waitcnt lgkmcnt(0)"), wx, Op("s_barrier")]
        if flavor == "steady" and p == 0 and nsc:
            post[xs].append(Op(f"s_mov_b32 s{S_AFTER}, 0"))
        pre[xs] += self.frag_read(self.vA(4), 0, p, 4)
        span = 5 * nm - 2 - xs
        m0_slots = set()

        def place(slot, op):
            """A copy needs one wait state between the write of m0 and its use: the MFMA of the slot is
            that instruction (m0 setup in front of it, the copy right behind)."""
            if len(op) == 3 and op[1].text == "s_nop 0" and not ({"nodma", "dmaonce", "m0nop"} & self.lab):
                assert slot not in m0_slots
                m0_slots.add(slot)
                pre[slot].append(op[0])
                post[slot].insert(0, op[2])
            else:
                post[slot] += op
        for n, op in enumerate(xops):
            place(xs + n * span // len(xops), op)
        post[5 * nm - 2] += adv_b
        pre[2 * nm] += self.frag_read(self.vA(5), 0, p, 5)
        pre[3 * nm] += self.frag_read(self.vA(6), 0, p, 6)
        pre[4 * nm] += self.frag_read(self.vA(7), 0, p, 7)
        # the next step's scale group: (p == 1) it sits in the other buffer; it has been published by this
        # step's X when its copy leads the X group of the step before, else by this step's Y
        sc_early = early and self.fp4 and (p == 0 or self.earlysc)
        sc_flip = [Op(f"v_xor_b32 v240, {SCBUF}, v240"), Op(f"v_xor_b32 v241, {SCBUF}, v241")] if (self.fp4 and p == 1 and prefetch) else []
        if early:
            er = []
            for jb in range(4):
                er += self.frag_read(self.vB(q, jb), 1, q, jb)
            if sc_early:
                post[xs] += sc_flip
                er += self.scale_reads(q, 1 if p == 0 else 0)
            e0, e1 = xs + 1, 5 * nm - 1
            for n, r in enumerate(er):
                post[e0 + n * (e1 - e0) // len(er)].append(r)
        # Y
        wy = WaitVm(("X", -1), keys)
        pre[tail0] += [Op("s_waitcnt lgkmcnt(0)"), wy, Op("s_barrier")]
        tail = total - tail0
        if prefetch:
            lds = []
            if not sc_early:
                post[tail0] += sc_flip
            for jb in range(4 if early else 0, 8):
                lds += self.frag_read(self.vB(q, jb), 1, q, jb)
            if self.fp4 and not sc_early:
                lds += self.scale_reads(q, 1 if p == 0 else 0)
            lds += self.frag_read(self.vA(0), 0, q, 0)
            span = tail // 2
            for n, l in enumerate(lds):
                post[tail0 + n * span // len(lds)].append(l)
            # A fragments 1 and 2 of the next step go where row blocks 5 and 6 read from: behind those
            a1 = max(tail0 + tail // 2, 6 * nm)
            a2 = max(tail0 + tail * 5 // 6, 7 * nm)
            post[a1] += self.frag_read(self.vA(1), 0, q, 1)
            post[a2] += self.frag_read(self.vA(2), 0, q, 2)
        for n, op in enumerate(a_hi):
            place(tail0 + n * (tail - 2) // len(a_hi), op)
        post[total - 2] += adv_a
        body = []
        for m in range(total):
            body += pre[m]
            body.append(self.mfma(p, m // nm, m % nm, first0))
            body += post[m]
        return out + self.lgkm_pass(body, pending0 if pending0 is not None else self.pending_at_step_start(p))

    # ---- LDS read completion -----------------------------------------------------------------------------
    @staticmethod
    def _vregs(tok):
        m = re.fullmatch(r"v\[(\d+):(\d+)\]", tok)
        if m:
            return set(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.fullmatch(r"v(\d+)", tok)
        return {int(m.group(1))} if m else set()

    def pending_at_step_start(self, p):
        """What a step may find in flight when it follows a step that prefetched for it: everything but
        A fragments 1 and 2 is older than those four reads."""
        older = set(range(self.vB(p, 0), self.vB(p, 0) + 64)) | set(range(self.vA(0), self.vA(0) + 8))
        if self.fp4:
            older |= set(range(self.scA(p, 0), self.scA(p, 0) + 16))
        a1, a2 = self.vA(1), self.vA(2)
        return [older, set(range(a1, a1 + 4)), set(range(a1 + 4, a1 + 8)), set(range(a2, a2 + 4)), set(range(a2 + 4, a2 + 8))]

    @classmethod
    def read_dests(cls, ops):
        return [cls._vregs(o.text.split()[1].rstrip(",")) for o in ops if isinstance(o, Op) and o.text.startswith("ds_read")]

    def lgkm_pass(self, ops, pending):
        """LDS reads complete in issue order; s_waitcnt lgkmcnt(n) lets the n youngest stay in flight.  Walks
        the instructions of a step and puts such a wait in front of every instruction that reads a register an
        LDS read in flight is going to write (the explicit lgkmcnt(0) in front of the barriers stay: they keep
        a wave from declaring LDS rows free that its own reads have not left yet)."""
        pending = list(pending)
        out = []
        for o in ops:
            if isinstance(o, WaitVm):
                out.append(o)
                continue
            t = o.text
            if t.startswith("ds_read"):
                pending.append(self._vregs(t.split()[1].rstrip(",")))
            elif t.startswith("s_waitcnt lgkmcnt("):
                n = int(t[t.index("(") + 1:t.index(")")])
                pending = pending[len(pending) - n:] if n else []
            elif t.startswith("v_") or t.startswith("global_"):
                # (every vector register the instruction names, its destination included: writing a register
                # that an LDS read in flight is about to overwrite would be just as wrong)
                srcs = set()
                for x in t.split()[1:]:
                    srcs |= self._vregs(x.rstrip(","))
                hit = max((k for k, d in enumerate(pending) if d & srcs), default=-1)
                if hit >= 0:
                    n = min(15, len(pending) - 1 - hit)
                    out.append(Op(f"s_waitcnt lgkmcnt({n})"))
                    pending = pending[len(pending) - n:] if n else []
            out.append(o)
        return out

    # ---- the whole K loop of one tile -------------------------------------------------------------------
    def prologue(self):
        out = []
        if self.fp4:
            for op in self.scale_dma(False, ("Y", -2)):
                out += op
        xb = ("XB", -1) if self.earlyb else ("X", -1)
        for st, tags in ((0, (("Y", -2), ("Y", -2), ("Y", -2), ("Y", -2))), (1, (xb, ("X", -1), ("X", -1), ("Y", -1)))):
            ops = self.dma(st, False, None)
            for grp, idx in zip(tags, ((8, 9, 12, 13), (10, 11, 14, 15), (0, 1, 4, 5), (2, 3, 6, 7))):   # B lo, B hi, A lo, A hi: the order the steps use
                for n in idx:
                    ops[n][-1].vm = grp
                    out += ops[n]
            out += self.dma_advance()
        out += [WaitVm(("Y", -2), {"a": 16}), Op("s_barrier")]
        return out

    def entry_reads(self):
        out = []
        if self.fp4:
            out += [Op(f"v_add_u32 v240, s{S_SCIN}, v232"), Op(f"v_add_u32 v241, s{S_SCIN}, v233")]
        for j in range(8):
            out += self.frag_read(self.vB(0, j), 1, 0, j)
        if self.fp4:
            out += self.scale_reads(0, 0)
        for t in range(3):
            out += self.frag_read(self.vA(t), 0, 0, t)
        return out

    def parts(self):
        """the pieces of the program, each a list of Op / WaitVm"""
        fp4 = self.fp4
        P = {}
        setup = [Op("; ==== 4-wave 256x256 K loop ===="),
                 Op(f"s_mov_b64 s[{S_CA}:{S_CA + 1}], %[A]"), Op(f"s_mov_b64 s[{S_CB}:{S_CB + 1}], %[B]"),
                 Op(f"s_mov_b64 s[{S_CROW}:{S_CROW + 1}], %[cprev]")]
        if fp4:
            setup += [Op(f"s_mov_b64 s[{S_CSA}:{S_CSA + 1}], %[mxa]"), Op(f"s_mov_b64 s[{S_CSB}:{S_CSB + 1}], %[mxb]"),
                      Op(f"s_mov_b32 s{S_SCIN}, %[scbuf]"), Op(f"s_mov_b32 s{S_SCN}, %[scbuf]")]
        P["setup"] = setup
        P["prologue"] = self.prologue()
        # later tiles: steps 0 and 1 (and scale group 0) were requested during the previous tile
        resume = [Op(f"s_add_u32 s{S_CA}, s{S_CA}, 256"), Op(f"s_addc_u32 s{S_CA + 1}, s{S_CA + 1}, 0"),
                  Op(f"s_add_u32 s{S_CB}, s{S_CB}, 256"), Op(f"s_addc_u32 s{S_CB + 1}, s{S_CB + 1}, 0")]
        if fp4:
            resume += [Op(f"s_add_u32 s{S_CSA}, s{S_CSA}, 16"), Op(f"s_addc_u32 s{S_CSA + 1}, s{S_CSA + 1}, 0"),
                       Op(f"s_add_u32 s{S_CSB}, s{S_CSB}, 16"), Op(f"s_addc_u32 s{S_CSB + 1}, s{S_CSB + 1}, 0"),
                       Op(f"s_xor_b32 s{S_SCN}, s{S_SCN}, {SCBUF}")]
        P["resume"] = resume
        # (either way s79 now names the buffer the NEXT scale group goes to)
        P["entry_fe"] = self.scale_reads_epi() if self.scaled_epi else []
        P["entry"] = [Op(f"s_mov_b32 s{S_AFTER}, 1")] + self.entry_reads()
        # (step 0 of a tile follows the entry reads: exactly those may be in flight)
        P["first0"] = self.step(0, False, True, "first0", self.read_dests(P["entry"]))
        P["first0_fe"] = self.step(0, False, True, "first0_fe", self.read_dests(P["entry_fe"] + P["entry"]))
        # (the same with fp16 results: %[fe] = 2)
        P["first0_fe16"] = self.step(0, False, True, "first0_fe16", self.read_dests(P["entry_fe"] + P["entry"]))
        P["first1"] = self.step(1, False, True, "first1")
        P["steady0"] = self.step(0, False, True)
        P["steady1"] = self.step(1, False, True)
        # the copy cursors move on to the next tile
        last_pre = [Op(f"s_mov_b64 s[{S_CA}:{S_CA + 1}], %[An]"), Op(f"s_mov_b64 s[{S_CB}:{S_CB + 1}], %[Bn]")]
        if fp4:
            last_pre += [Op(f"s_mov_b64 s[{S_CSA}:{S_CSA + 1}], %[mxan]"), Op(f"s_mov_b64 s[{S_CSB}:{S_CSB + 1}], %[mxbn]")]
        P["last_pre"] = last_pre
        P["last0"] = self.step(0, True, True)
        P["last1"] = self.step(1, True, False)
        # the accumulators may be read by vector instructions 18 wait states after the last MFMA
        end = [Op("s_nop 7"), Op("s_nop 7"), Op("s_nop 7")]
        if fp4:
            # the buffer that holds the next tile's first scale group
            end.append(Op(f"s_xor_b32 %[scbuf], s{S_SCN}, {SCBUF}"))
        P["end"] = end
        self.solve(P)
        return P

    # ---- text ---------------------------------------------------------------------------------------------
    def wait_text(self, w):
        """the instructions of one wait site: a single s_waitcnt, or a choice by the history flags"""
        vals = w.vals
        distinct = sorted(set(vals.values()))
        if len(distinct) == 1:
            return [f"s_waitcnt vmcnt({distinct[0]})"]
        self.lbl += 1
        L = lambda x: f"W4_W{self.lbl}{x}_%="
        out = []
        if set(vals) == {"s", "f"}:
            out += [f"s_cmp_lg_u32 s{S_AFTER}, 0", f"s_cbranch_scc1 {L('f')}", f"s_waitcnt vmcnt({vals['s']})", f"s_branch {L('z')}",
                    f"{L('f')}:", f"s_waitcnt vmcnt({vals['f']})", f"{L('z')}:"]
            return out
        order = [("a", "%[first]"), ("d", "%[fe]"), ("b", "%[nst]")]
        for k, flag in order:
            if k in vals:
                out += [f"s_cmp_lg_u32 {flag}, 0", f"s_cbranch_scc1 {L(k)}"]
        if "c" in vals:
            out += [f"s_waitcnt vmcnt({vals['c']})", f"s_branch {L('z')}"]
        for k, flag in order:
            if k in vals:
                out += [f"{L(k)}:", f"s_waitcnt vmcnt({vals[k]})", f"s_branch {L('z')}"]
        out.append(f"{L('z')}:")
        return out

    def lines(self, ops, keep_dma=False):
        out = []
        for o in ops:
            if isinstance(o, WaitVm):
                ls = self.wait_text(o)
            else:
                ls = [o.text]
            for s in ls:
                if "nomfma" in self.lab and s.startswith("v_mfma"):
                    continue
                if ("nodma" in self.lab or ("dmaonce" in self.lab and not keep_dma)) and s.startswith("global_load_lds"):
                    continue
                if "noread" in self.lab and s.startswith("ds_read"):
                    continue
                if "nobar" in self.lab and s.startswith("s_barrier"):
                    continue
                if "novm" in self.lab and s.startswith("s_waitcnt vmcnt"):
                    continue
                if "nolgk" in self.lab and s.startswith("s_waitcnt lgkmcnt"):
                    continue
                if "nostore" in self.lab and s.startswith("global_store"):
                    continue
                if ({"noscale", "noscaleread"} & self.lab) and s.startswith("ds_read_u16"):
                    continue
                if ({"noscale", "noscaledma"} & self.lab) and s.startswith("global_load_lds_dwordx4 v23") and s[27] in "4567":
                    continue
                out.append(s)
        return out

    def program(self):
        P = self.parts()
        T = lambda name: self.lines(P[name])
        out = T("setup")
        out += ["s_cmp_eq_u32 %[first], 0", "s_cbranch_scc1 W4_RESUME%="]
        out += self.lines(P["prologue"], keep_dma=True) + ["s_branch W4_ENTRY%=", "W4_RESUME%=:"] + T("resume") + ["W4_ENTRY%=:"]
        if self.scaled_epi:
            # (22 fragment reads follow: a wait for "at most 15 outstanding" then covers these 16)
            out += ["s_cmp_eq_u32 %[fe], 0", "s_cbranch_scc1 W4_NOSC%="] + T("entry_fe") + ["W4_NOSC%=:"]
        out += T("entry")
        out += ["s_cmp_lg_u32 %[fe], 0", "s_cbranch_scc1 W4_FE%="]
        out += T("first0") + ["s_branch W4_FIRST1%=", "W4_FE%=:", "s_cmp_eq_u32 %[fe], 2", "s_cbranch_scc1 W4_FE16%="]
        out += T("first0_fe") + ["s_branch W4_FIRST1%=", "W4_FE16%=:"] + T("first0_fe16") + ["W4_FIRST1%=:"] + T("first1")
        out += [f"s_sub_u32 s{S_CNT}, %[kh], 2", f"s_cmp_eq_u32 s{S_CNT}, 0", "s_cbranch_scc1 W4_LAST%=", "W4_LOOP%=:"]
        out += T("steady0") + T("steady1")
        out += [f"s_sub_u32 s{S_CNT}, s{S_CNT}, 1", f"s_cmp_lg_u32 s{S_CNT}, 0", "s_cbranch_scc1 W4_LOOP%=", "W4_LAST%=:"]
        out += T("last_pre") + T("last0") + T("last1") + T("end")
        return out

    def text(self):
        return "".join(f'  "{l}\\n\\t"\n' for l in self.program())

    # ---- wait counts: solved and checked by replay -----------------------------------------------------------
    def replay(self, P, visit):
        """Replays the vector-memory operations of every history a tile can have (first tile of the
        workgroup; after a tile whose epilogue ran as compiled code with 32 stores, or with an unknown
        number -- tried with none and with many; after a tile whose epilogue is fused into this one) for
        tiles of 4, 6, 8 and 10 K steps, three tiles in a row, and calls visit(wait, history key, number of
        operations issued after the awaited group, where) at every wait."""
        def run(seq):
            """seq: list of (part name, step number, history key or None)"""
            q = []       # tags in issue order
            for name, step, hist in seq:
                if name == "cstores":
                    q += [("CST", step)] * hist
                    continue
                for o in P[name]:
                    if isinstance(o, WaitVm):
                        grp = (o.awaits[0], o.awaits[1] + step)
                        key = hist if hist in o.vals else ("s" if "s" in o.vals else None)
                        assert key is not None, (name, step, hist, o.vals)
                        idx = max((i for i, t in enumerate(q) if t == grp), default=-1)
                        assert idx >= 0, f"{self.kind}: {name} step {step} waits for {grp}, which nobody issued"
                        visit(o, key, len(q) - 1 - idx, f"{self.kind}: {name} step {step} history {hist}: wait for {grp}")
                    elif o.vm is not None:
                        q.append((o.vm[0], o.vm[1] + step))

        def tile(base, ksteps, hist0, fe_part="first0_fe"):
            """parts of one tile whose step 0 is number `base`"""
            t = [(fe_part if hist0 == "d" else "first0", base, hist0), ("first1", base + 1, hist0)]
            h = "f"
            for it in range(2, ksteps - 2, 2):
                t += [("steady0", base + it, h), ("steady1", base + it + 1, "s")]
                h = "s"
            t += [("last0", base + ksteps - 2, h), ("last1", base + ksteps - 1, "s")]
            return t

        for k in (4, 6, 8, 10):
            for hist, nstores, fe_part in (("b", NST, None), ("c", 0, None), ("c", 50, None), ("d", 0, "first0_fe"), ("d", 0, "first0_fe16")):
                seq = [("prologue", 0, "a")] + tile(0, k, "a")
                seq += [("cstores", k, nstores)] + tile(k, k, hist, fe_part)
                seq += [("cstores", 2 * k, NST)] + tile(2 * k, k, "b")
                run(seq)

    def solve(self, P):
        """vmcnt counts loads and stores in issue order: a wait for a group of copies may leave as many
        operations in flight as were issued after that group -- in EVERY history that reaches the wait.
        Fills in the counts that the steps left open with the smallest such number."""
        found = {}

        def visit(o, key, younger, where):
            if o.vals[key] is None:
                found[(id(o), key)] = min(found.get((id(o), key), 63), younger)
        self.replay(P, visit)
        for part in P.values():
            for o in part:
                if isinstance(o, WaitVm):
                    for key in o.vals:
                        if o.vals[key] is None:
                            o.vals[key] = found.get((id(o), key), 0)    # (a history that never reaches the wait: drain)

    def check(self):
        """Replays every history (see replay) and checks at every wait that the number it allows in flight
        does not exceed the number of operations issued after the awaited group.  Returns the slack per
        wait site."""
        P = self.parts()
        worst = {}

        def visit(o, key, younger, where):
            n = o.vals[key]
            assert n <= younger, f"{where}: vmcnt({n}), only {younger} younger operations exist"
            site = (where.split(":")[1].split(" step")[0].strip(), o.awaits, key)
            worst[site] = min(worst.get(site, 99), younger - n)
        self.replay(P, visit)
        return worst


def clobbers(kind):
    """registers the statement writes that are not operands of it"""
    v = list(range(192)) + [240, 241] if kind == "fp4" else list(range(160))
    names = [f"v{i}" for i in v] + [f"a{i}" for i in range(256)] + [f"s{i}" for i in range(70, 90)]
    names += ["memory", "vcc", "scc", "m0"]
    lines = []
    for i in range(0, len(names), 16):
        lines.append("  " + ", ".join(f'"{n}"' for n in names[i:i + 16]))
    return ",\n".join(lines) + "\n"


def main():
    what = sys.argv[1]
    if what == "clobbers":
        sys.stdout.write(clobbers(sys.argv[2]))
        return
    if what == "check":
        for kind in F8_KINDS + ("fp4", "bf16", "f16", "i8"):
            w = Gen(kind).check()
            print(kind, "ok; smallest slack per wait site:", min(w.values()), "largest:", max(w.values()))
        return
    g = Gen(what, [x for x in os.environ.get("W4GEN_LAB", "").split(",") if x])
    g.check()
    sys.stdout.write(g.text())


if __name__ == "__main__":
    main()
