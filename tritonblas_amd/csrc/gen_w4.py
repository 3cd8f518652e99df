#!/usr/bin/env python3
"""Writes the hand-scheduled K loop of the 4-wave 256x256 tile kernels (gemm_w4.h) as inline-assembly text.

    python3 gen_w4.py fp8 > w4_kloop_fp8.inc        (also: fp4, bf16, f16)
    python3 gen_w4.py clobbers > w4_clobbers.inc

One workgroup = 4 waves (one per SIMD), wave (wm, wn) owns the 128x128 quarter of a 256x256 output
tile: 8x8 MFMA tiles of 16x16, i.e. 256 accumulator registers a[0:255]; acc(i, j) of A row block i and
B row block j sits in a[(8i+j)*4 .. +3].  A K step is 128 bytes of every operand row (128 FP8 values,
256 FP4 values or 64 16-bit values); LDS holds two stages of 64 KB: stage s at s*65536, A rows at +0, B rows at +32768,
row r at r*128 with its eight 16-byte chunks XOR-swizzled (the layout the 8-wave kernels use).  FP4
adds two 8 KB buffers of E8M0 scales behind the stages (16 scale bytes per row = two K steps).

The text below is the code of ONE asm statement that runs the whole K loop of one output tile:

  entry      (first tile of the workgroup only) copies of K steps 0 and 1 and of scale group 0
  per K step eight row blocks of MFMAs (row block i multiplies A fragment i with the eight B fragments);
             the A fragment of row block i+3 is requested when row block i starts (four fragment
             buffers), the B fragments of the next step sit in the other of two B register sets;
             in front of row block 5 all LDS reads of the step have been issued:
             lgkmcnt(0), vmcnt(0) (next step's copies have landed), s_barrier, and behind it, between
             the 24 MFMAs of row blocks 5..7, the copies of step +2 into the stage just freed and the
             reads of the next step's B fragments, scales and first A fragments
  last two   the copies go to the NEXT tile's first two K steps (the caller passes the next tile's
  K steps    addresses, or the same tile's again when there is none), so the copy pipeline never drains
             between tiles; no fragments are prefetched across the tile boundary.

K must be a multiple of two K steps (the loop body is the even step followed by the odd step).

Register map (VGPR):  0..127  B fragment sets 0/1 (8 fragments x 8 registers each)
                      128..159 A fragment buffers 0..3
                      160..191 FP4 scale registers, set p: A rows 160+16p+i, B rows 168+16p+j
                      192..207 inputs: byte offsets of this tile's copies (A 192+i, B 200+i, i = copy instruction)
                      208..223 inputs: the same for the next tile
                      224..231 inputs: fragment read addresses (A lo, A hi, B lo, B hi) for stage 0, then stage 1
                      232..237 inputs: scale read addresses (A, B), scale copy offsets (A, B) now and next
                      240, 241 scratch: scale read addresses of the current scale buffer
SGPR 70..82 are scratch (copy cursors, loop counter, scale buffer toggle, first-step flag).
"""
import sys

STAGE = 65536
BOFF = 32768
SC0 = 131072          # scale buffers behind the two stages
SCBUF = 8192
NST = 32              # stores per wave of the fast epilogue (256x256 16-bit values, 16 bytes per lane and store)
import os
BND = int(os.environ.get("W4GEN_BND", "5"))   # the K-step boundary sits in front of this row block

S_CA, S_CB, S_CSA, S_CSB, S_CNT, S_SCN, S_T, S_SCIN, S_FIRST = 70, 72, 74, 76, 78, 79, 80, 81, 82


class Gen:
    def __init__(self, kind, dma_every=1, lab=()):
        self.kind = kind                # "fp8" | "fp4" | "bf16" | "f16"
        self.fp4 = kind == "fp4"        # (the only kind with E8M0 scale operands)
        self.out = []
        self.nm = 8 if kind == "fp8" else 16      # MFMAs per row block (FP8: one of K = 128 per fragment pair; others: two half-K ones)
        self.dma_every = dma_every
        self.lbl = 0
        # how far (in MFMAs) into row blocks 1 and 5 the two sync points of a K step sit
        self.xoff = int(os.environ.get("W4GEN_XOFF", str(self.nm // 2)))
        self.yoff = int(os.environ.get("W4GEN_YOFF", str(self.nm // 2)))
        # measurement builds (W4GEN_LAB=nomfma,nodma,noread,nobar): leave one kind of instruction out to time
        # the rest; results are then meaningless
        self.lab = set(lab)

    def e(self, s):
        if "nomfma" in self.lab and s.startswith("v_mfma"):
            return
        if "nodma" in self.lab and s.startswith("global_load_lds"):
            return
        if "noread" in self.lab and s.startswith("ds_read"):
            return
        if "nobar" in self.lab and s.startswith("s_barrier"):
            return
        if "novm" in self.lab and s.startswith("s_waitcnt vmcnt"):
            return
        if "nolgk0" in self.lab and s == "s_waitcnt lgkmcnt(0)":
            return
        if "nolgk" in self.lab and s.startswith("s_waitcnt lgkmcnt"):
            return
        self.out.append(s)

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
        return [f"ds_read_b128 v[{dst}:{dst + 3}], v{self.fa(op, 0, stage)} offset:{t * 2048}",
                f"ds_read_b128 v[{dst + 4}:{dst + 7}], v{self.fa(op, 1, stage)} offset:{t * 2048}"]

    def scale_reads(self, p, half):
        """E8M0 bytes of one K step for all row blocks: two bytes (k slices 0, 1) per lane and row block"""
        r = []
        for i in range(8):
            r.append(f"ds_read_u16 v{self.scA(p, i)}, v240 offset:{i * 256 + half * 8}")
        for j in range(8):
            r.append(f"ds_read_u16 v{self.scB(p, j)}, v241 offset:{j * 256 + half * 8}")
        return r

    def dma(self, stage, nxt):
        """the 16 LDS-direct copies of one K step (A then B), each as [m0 setup, wait state, load]"""
        ops = []
        base = 208 if nxt else 192
        for op, cur in ((0, S_CA), (1, S_CB)):
            for i in range(8):
                imm = stage * STAGE + op * BOFF + i * 4096
                ops.append([f"s_add_u32 m0, %[wl], {imm}", "s_nop 0",
                            f"global_load_lds_dwordx4 v{base + op * 8 + i}, s[{cur}:{cur + 1}]"])
        return ops

    def dma_advance(self):
        return [f"s_add_u32 s{S_CA}, s{S_CA}, 128", f"s_addc_u32 s{S_CA + 1}, s{S_CA + 1}, 0",
                f"s_add_u32 s{S_CB}, s{S_CB}, 128", f"s_addc_u32 s{S_CB + 1}, s{S_CB + 1}, 0"]

    def scale_dma(self, nxt):
        """copy of one scale group (16 bytes per row, A rows then B rows) into the buffer s79 names, then toggle it"""
        va, vb = (236, 237) if nxt else (234, 235)
        return [[f"s_add_u32 s{S_T}, %[wl], s{S_SCN}", f"s_add_u32 m0, s{S_T}, {SC0}", "s_nop 0",
                 f"global_load_lds_dwordx4 v{va}, s[{S_CSA}:{S_CSA + 1}]"],
                [f"s_add_u32 m0, s{S_T}, {SC0 + 4096}", "s_nop 0",
                 f"global_load_lds_dwordx4 v{vb}, s[{S_CSB}:{S_CSB + 1}]",
                 f"s_xor_b32 s{S_SCN}, s{S_SCN}, {SCBUF}",
                 f"s_add_u32 s{S_CSA}, s{S_CSA}, 16", f"s_addc_u32 s{S_CSA + 1}, s{S_CSA + 1}, 0",
                 f"s_add_u32 s{S_CSB}, s{S_CSB}, 16", f"s_addc_u32 s{S_CSB + 1}, s{S_CSB + 1}, 0"]]

    def mfma(self, p, i, slot):
        """MFMA number `slot` of row block i: B fragment first (its rows become the output rows a lane holds)"""
        if self.kind == "fp8":
            j = slot
            acc = (i * 8 + j) * 4
            b, a = self.vB(p, j), self.vA(i)
            return f"v_mfma_f32_16x16x128_f8f6f4 a[{acc}:{acc + 3}], v[{b}:{b + 7}], v[{a}:{a + 7}], a[{acc}:{acc + 3}]"
        # two MFMAs per accumulator and K step, k slice outermost so that the same accumulator comes up
        # again only eight instructions later
        ks, j = slot // 8, slot % 8
        acc = (i * 8 + j) * 4
        b, a = self.vB(p, j) + 4 * ks, self.vA(i) + 4 * ks
        if self.kind in ("bf16", "f16"):
            return f"v_mfma_f32_16x16x32_{self.kind} a[{acc}:{acc + 3}], v[{b}:{b + 3}], v[{a}:{a + 3}], a[{acc}:{acc + 3}]"
        return (f"v_mfma_scale_f32_16x16x128_f8f6f4 a[{acc}:{acc + 3}], v[{b}:{b + 3}], v[{a}:{a + 3}], a[{acc}:{acc + 3}], "
                f"v{self.scB(p, j)}, v{self.scA(p, i)} op_sel:[{ks},{ks},0] op_sel_hi:[0,0,0] cbsz:4 blgp:4")

    # ---- one K step -------------------------------------------------------------------------------
    def wait_vm(self, n, n_stores, n_cons):
        """s_waitcnt vmcnt(n) in the steady state.  While s82 is set (first K steps of a tile) the previous
        tile's epilogue stores are younger than the copies waited for: with %[nst] they are exactly 32 per
        wave and the wait allows for them (n_stores), otherwise it assumes none (n_cons)."""
        self.lbl += 1
        f, g, d = (f"W4_V{x}{self.lbl}_%=" for x in "FGD")
        return [f"s_cmp_lg_u32 s{S_FIRST}, 0", f"s_cbranch_scc1 {f}", f"s_waitcnt vmcnt({n})", f"s_branch {d}",
                f"{f}:", "s_cmp_lg_u32 %[nst], 0", f"s_cbranch_scc1 {g}", f"s_waitcnt vmcnt({n_cons})", f"s_branch {d}",
                f"{g}:", f"s_waitcnt vmcnt({n_stores})", f"{d}:"]

    def step(self, p, nxt, prefetch):
        """K step in stage p (= B set p, scale set p).  nxt: the copies issued in this step read the
        next tile.  prefetch: request the following step's fragments in the tail.

        Two sync points (wait + s_barrier) per step, each followed by copies of step +2 into LDS that
        every wave has just declared free:
          X, in front of row block 1: this step's B fragments and A fragments 0..3 are in registers
             -> B half of the stage and the A rows of row blocks 0..3 ("A lo") take step +2;
             it also publishes "A hi" of THIS step (row blocks 4..7), which is read from here on;
          Y, in front of row block 5 (the step boundary): A fragments 4..7 are in registers
             -> "A hi" takes step +2; it publishes B and "A lo" of the NEXT step for the tail's reads.
        Every copy is therefore waited for one and a half K steps after it was issued, and two to
        three bursts overlap in time: one burst per step that has to land within one step leaves the
        L2 -> LDS path idle for the latency of its first byte and then stalls the MFMAs at the wait.
        vmcnt counts in issue order, so each wait names how many younger copies may stay in flight."""
        nm = self.nm
        total = 8 * nm
        self.e(f"; ---- K step, stage {p}{' (copies: next tile)' if nxt else ''}{'' if prefetch else ' (last of the tile)'}")
        pre = [[] for _ in range(total)]      # in front of MFMA slot m
        post = [[] for _ in range(total)]     # behind it
        ops = self.dma(p, nxt)
        lo = [ops[i] for i in (0, 1, 4, 5)]                 # A rows of row blocks 0..3 (both wave rows)
        hi = [ops[i] for i in (2, 3, 6, 7)]
        ops_b = ops[8:]
        adv = self.dma_advance()
        adv_a, adv_b = adv[:2], adv[2:]
        sc = self.scale_dma(nxt) if (self.fp4 and p == 0) else []
        nx = len(ops_b) + len(lo) + len(sc)                # copies issued behind X of this step
        nx_other = 12 + (2 if (self.fp4 and p == 1) else 0)   # ... behind X of the neighbouring steps
        # row block 0
        pre[0] += self.frag_read(self.vA(3), 0, p, 3)
        pre[0].append("s_waitcnt lgkmcnt(6)")
        # X: part of the way into row block 1, so that the read of A fragment 3 (requested when row block 0
        # started) has had time to return before lgkmcnt(0) asks for it
        xs = nm + self.xoff
        # (X of step 0: nothing of this tile may be assumed younger than the stores; X of step 1: the
        # steady-state count already demands that the stores are done)
        pre[xs] += ["s_waitcnt lgkmcnt(0)"] + self.wait_vm(nx_other + 4, nx_other + 4 + NST, 0 if p == 0 else nx_other + 4) + ["s_barrier"]
        if p == 1:
            post[xs].append(f"s_mov_b32 s{S_FIRST}, 0")
        pre[xs] += self.frag_read(self.vA(4), 0, p, 4)
        xops = ops_b + lo + sc
        span = 5 * nm - 2 - xs
        for n, op in enumerate(xops):
            post[xs + n * span // len(xops)] += op
        post[5 * nm - 2] += adv_b
        pre[2 * nm] += self.frag_read(self.vA(5), 0, p, 5)
        pre[3 * nm] += self.frag_read(self.vA(6), 0, p, 6)
        pre[4 * nm] += self.frag_read(self.vA(7), 0, p, 7)
        # (A fragment 4 was requested at X; fragments 5, 6, 7 are younger)
        pre[4 * nm].append("s_waitcnt lgkmcnt(6)")
        # Y
        tail0 = BND * nm + self.yoff
        if p == 0:
            pre[tail0] += ["s_waitcnt lgkmcnt(0)"] + self.wait_vm(nx + 4, nx + 4 + NST, nx) + ["s_barrier"]
        else:
            pre[tail0] += ["s_waitcnt lgkmcnt(0)", f"s_waitcnt vmcnt({nx + 4})", "s_barrier"]
        tail = total - tail0
        q = p ^ 1
        if prefetch:
            lds = []
            if self.fp4 and p == 1:
                # the next step opens a new scale group: it sits in the other buffer
                post[tail0] += [f"v_xor_b32 v240, {SCBUF}, v240", f"v_xor_b32 v241, {SCBUF}, v241"]
            for j in range(8):
                lds += self.frag_read(self.vB(q, j), 1, q, j)
            if self.fp4:
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
        for n, op in enumerate(hi):
            post[tail0 + n * (tail - 2) // len(hi)] += op
        post[total - 2] += adv_a
        for m in range(total):
            for l in pre[m]:
                self.e(l)
            self.e(self.mfma(p, m // nm, m % nm))
            for l in post[m]:
                self.e(l)

    # ---- the whole K loop of one tile -------------------------------------------------------------------
    def kloop(self):
        e = self.e
        fp4 = self.fp4
        e("; ==== 4-wave 256x256 K loop ====")
        e(f"s_mov_b64 s[{S_CA}:{S_CA + 1}], %[A]")
        e(f"s_mov_b64 s[{S_CB}:{S_CB + 1}], %[B]")
        if fp4:
            e(f"s_mov_b64 s[{S_CSA}:{S_CSA + 1}], %[mxa]")
            e(f"s_mov_b64 s[{S_CSB}:{S_CSB + 1}], %[mxb]")
            e(f"s_mov_b32 s{S_SCIN}, %[scbuf]")
            e(f"s_mov_b32 s{S_SCN}, %[scbuf]")
        e("s_cmp_eq_u32 %[first], 0")
        e("s_cbranch_scc1 W4_RESUME%=")
        # first tile of the workgroup: fill both stages (and the first scale group)
        if fp4:
            for op in self.scale_dma(False):
                for l in op:
                    e(l)
        for st in (0, 1):
            ops = self.dma(st, False)
            for n in (8, 9, 10, 11, 12, 13, 14, 15, 0, 1, 4, 5, 2, 3, 6, 7):   # B, A lo, A hi: the order the steps use
                for l in ops[n]:
                    e(l)
            for l in self.dma_advance():
                e(l)
        e("s_waitcnt vmcnt(16)")
        e("s_barrier")
        e("s_branch W4_ENTRY%=")
        e("W4_RESUME%=:")
        # later tiles: steps 0 and 1 (and scale group 0) were requested during the previous tile
        e(f"s_add_u32 s{S_CA}, s{S_CA}, 256")
        e(f"s_addc_u32 s{S_CA + 1}, s{S_CA + 1}, 0")
        e(f"s_add_u32 s{S_CB}, s{S_CB}, 256")
        e(f"s_addc_u32 s{S_CB + 1}, s{S_CB + 1}, 0")
        if fp4:
            e(f"s_add_u32 s{S_CSA}, s{S_CSA}, 16")
            e(f"s_addc_u32 s{S_CSA + 1}, s{S_CSA + 1}, 0")
            e(f"s_add_u32 s{S_CSB}, s{S_CSB}, 16")
            e(f"s_addc_u32 s{S_CSB + 1}, s{S_CSB + 1}, 0")
            e(f"s_xor_b32 s{S_SCN}, s{S_SCN}, {SCBUF}")
        e("W4_ENTRY%=:")
        e(f"s_mov_b32 s{S_FIRST}, 1")
        # (either way s79 now names the buffer the NEXT scale group goes to)
        if fp4:
            e(f"v_add_u32 v240, s{S_SCIN}, v232")
            e(f"v_add_u32 v241, s{S_SCIN}, v233")
        for j in range(8):
            for l in self.frag_read(self.vB(0, j), 1, 0, j):
                e(l)
        if fp4:
            for l in self.scale_reads(0, 0):
                e(l)
        for t in range(3):
            for l in self.frag_read(self.vA(t), 0, 0, t):
                e(l)
        for n in range(256):
            e(f"v_accvgpr_write_b32 a{n}, 0")
        e(f"s_sub_u32 s{S_CNT}, %[kh], 1")
        e(f"s_cmp_eq_u32 s{S_CNT}, 0")
        e("s_cbranch_scc1 W4_LAST%=")
        e("W4_LOOP%=:")
        self.step(0, False, True)
        self.step(1, False, True)
        e(f"s_sub_u32 s{S_CNT}, s{S_CNT}, 1")
        e(f"s_cmp_lg_u32 s{S_CNT}, 0")
        e("s_cbranch_scc1 W4_LOOP%=")
        e("W4_LAST%=:")
        # the copy cursors move on to the next tile
        e(f"s_mov_b64 s[{S_CA}:{S_CA + 1}], %[An]")
        e(f"s_mov_b64 s[{S_CB}:{S_CB + 1}], %[Bn]")
        if fp4:
            e(f"s_mov_b64 s[{S_CSA}:{S_CSA + 1}], %[mxan]")
            e(f"s_mov_b64 s[{S_CSB}:{S_CSB + 1}], %[mxbn]")
        self.step(0, True, True)
        self.step(1, True, False)
        # the accumulators may be read by vector instructions 18 wait states after the last MFMA
        e("s_nop 7")
        e("s_nop 7")
        e("s_nop 7")
        if fp4:
            # the buffer that holds the next tile's first scale group
            e(f"s_xor_b32 %[scbuf], s{S_SCN}, {SCBUF}")

    def text(self):
        return "".join(f'  "{l}\\n\\t"\n' for l in self.out)


def clobbers():
    names = [f"v{i}" for i in range(192)] + ["v240", "v241"] + [f"a{i}" for i in range(256)] + [f"s{i}" for i in range(70, 83)]
    names += ["memory", "vcc", "scc", "m0"]
    lines = []
    for i in range(0, len(names), 16):
        lines.append("  " + ", ".join(f'"{n}"' for n in names[i:i + 16]))
    return ",\n".join(lines) + "\n"


def main():
    what = sys.argv[1]
    if what == "clobbers":
        sys.stdout.write(clobbers())
        return
    import os
    every = int(os.environ.get("W4GEN_DMA_EVERY", "1" if what == "fp8" else "2"))
    g = Gen(what, every, [x for x in os.environ.get("W4GEN_LAB", "").split(",") if x])
    g.kloop()
    sys.stdout.write(g.text())


if __name__ == "__main__":
    main()
