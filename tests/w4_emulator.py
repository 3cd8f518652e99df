"""CPU replay of the generated K loop of the 4-wave kernels (tritonblas_amd/csrc/gen_w4.py): test infrastructure.

The K loop of gemm_w4.h is assembly text.  This module interprets that text for one wave -- scalar arithmetic,
branches, the address registers, every LDS-direct copy, LDS read, MFMA and store -- over a sequence of tiles of
one workgroup, with the operands the C++ side of gemm_w4.h would hand over (restated here: lane constants, tile
arguments, the history flags), and checks

* addresses: every copy reads inside the operand it belongs to (A, B, the FP4 scale matrices, the epilogue scale
  vectors), every LDS write and read stays inside the LDS area it is meant for, every store lands inside the
  previous tile of C and the wave's quarter of it is written exactly once;
* data flow: an LDS read only touches bytes whose copy has completed (a vmcnt wait that covers it, then a
  barrier) and a copy only overwrites bytes whose last read completed before the latest barrier; every MFMA
  multiplies fragment i of A with fragment j of B of the CURRENT tile and K step into accumulator (i, j), with
  the E8M0 bytes of exactly those rows and that K block.

It knows nothing about timing: it proves that the schedule is right for every order in which the hardware may
complete what the waits allow to be outstanding."""
import importlib.util
import os
import re

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
GEN = os.path.join(os.path.dirname(HERE), "tritonblas_amd", "csrc", "gen_w4.py")


def load_generator():
    spec = importlib.util.spec_from_file_location("gen_w4", GEN)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


LDS0 = 0                 # where the kernel's LDS array starts: the only __shared__ object of the kernel sits at offset 0 (the scale
                         # buffer switches XOR buffer sizes into absolute LDS addresses, which needs a 32 KB aligned start)
STAGE, BOFF, SC0 = 65536, 32768, 131072
MASK32, MASK64 = (1 << 32) - 1, (1 << 64) - 1


class Fail(AssertionError):
    pass


class Space:
    """one operand in (pretend) global memory"""
    def __init__(self, name, base, rows, stride, row_bytes):
        self.name, self.base, self.rows, self.stride, self.row_bytes = name, base, rows, stride, row_bytes

    @property
    def end(self):
        return self.base + (self.rows - 1) * self.stride + self.row_bytes

    def locate(self, addr, size):
        """(row, byte in row) of [addr, addr + size), which must lie inside one row"""
        off = addr - self.base
        row, col = divmod(off, self.stride)
        if off < 0 or row >= self.rows or col + size > self.row_bytes:
            return None
        return row, col


def b_tile_row(row):
    """the tile row that LDS row `row` of the B tile holds (gemm_w4.h: eight consecutive output columns per lane)"""
    rho = row & 127
    j, gg, e = rho >> 4, (rho >> 2) & 3, rho & 3
    return (row & 128) + (j >> 1) * 32 + gg * 8 + (j & 1) * 4 + e


class Problem:
    """Shapes, strides and base addresses of one GEMM, and the tiles one workgroup runs."""
    def __init__(self, kind, m, n, ksteps, tiles, pad=0, scales=True):
        self.kind, self.m, self.n, self.ksteps, self.tiles = kind, m, n, ksteps, tiles
        kb = ksteps * 128                           # bytes of K per operand row
        self.A = Space("A", 0x10_0000_0000, m, kb + pad, kb)
        self.B = Space("B", 0x20_0000_0000, n, kb + pad, kb)
        self.C = Space("C", 0x30_0000_0000, m, n * 2 + 2 * pad, n * 2)
        self.fp4 = kind == "fp4"
        self.scaled = kind in ("fp8", "e5m2", "i8") and scales
        mxb = ksteps * 8
        self.mxa = Space("mxa", 0x40_0000_0000, m, mxb + (pad // 16) * 16, mxb)
        self.mxb = Space("mxb", 0x50_0000_0000, n, mxb + (pad // 16) * 16, mxb)
        self.sa = Space("sa", 0x60_0000_0000, 1, 4 * m, 4 * m)
        self.sb = Space("sb", 0x70_0000_0000, 1, 4 * n, 4 * n)
        self.spaces = [self.A, self.B, self.mxa, self.mxb, self.sa, self.sb]


class Wave:
    """One wave of the workgroup: registers, the LDS shadow, the queues the waits refer to."""
    def __init__(self, gen, prob, wave, group, ragged_stores=7):
        self.gen, self.prob, self.wave = gen, prob, wave
        self.group = group   # the four waves of the workgroup (they share the LDS and run in step)
        self.kind = prob.kind
        self.ragged_stores = ragged_stores
        lane = np.arange(64, dtype=np.int64)
        self.lane = lane
        self.r, self.g = lane & 15, lane >> 4
        self.wm0, self.wn0 = (wave >> 1) * 128, (wave & 1) * 128
        l8 = lane >> 3
        self.c16 = ((lane & 7) ^ l8 ^ (wave & 1)) << 4
        self.pa = wave * 8 + l8
        self.pb = ((wave & 1) * 2 + (l8 >> 2)) * 8 + (wave >> 1) * 4 + (l8 & 3)
        self.sra = wave * 64 + lane
        self.srb = np.array([b_tile_row(int(x)) for x in self.sra])
        self.S = {}          # scalar registers by name ("s70", "m0", "scc") and bound operands ("%[A]")
        self.V = {}          # vector registers that hold addresses: number -> uint32[64]
        self.meta = {}       # vector register -> what an LDS read put there
        self.lds = group.lds  # LDS byte offset (4-byte granularity) -> dict(what=..., vm=entry, pub=bool), shared
        self.vmq = []        # vector memory operations in issue order: dict(done=bool, lds=[offsets])
        self.reads = 0       # LDS reads issued; the first `reads - outstanding` have completed
        self.outstanding = 0
        self.covered = 0     # number of reads that had completed at the latest barrier
        self.last_read = {}  # LDS offset -> sequence number of the last read of it
        self.stores = {}     # C address -> count
        self.step = None     # (tile index, K step) the MFMAs in flight belong to
        self.log = []

    # ---- operand restatement of gemm_w4.h ------------------------------------------------------------------
    def tile_args(self, t):
        p = self.prob
        m0, n0 = t[:2]
        it0 = t[2] if len(t) > 2 else 0          # a Stream-K piece starts at K step it0 of its tile
        rva, rvb = min(256, p.m - m0), min(256, p.n - n0)
        a = {"A": p.A.base + m0 * p.A.stride + it0 * 128, "B": p.B.base + n0 * p.B.stride + it0 * 128,
             "mxa": p.mxa.base + m0 * p.mxa.stride + it0 * 8, "mxb": p.mxb.base + n0 * p.mxb.stride + it0 * 8, "rva": rva, "rvb": rvb}
        off = []
        for i in range(8):
            off.append(np.minimum(i * 32 + self.pa, rva - 1) * p.A.stride + self.c16)
        for i in range(8):
            off.append(np.minimum(i * 32 + self.pb, rvb - 1) * p.B.stride + self.c16)
        a["off"] = off
        a["sca"] = np.minimum(self.sra, rva - 1) * p.mxa.stride
        a["scb"] = np.minimum(self.srb, rvb - 1) * p.mxb.stride
        return a

    def bind(self, ti, first, nst, fe, cprev, scbuf):
        """registers and operands of the statement for tile number ti (what the C++ loop computes)"""
        p, g = self.prob, self.gen
        tiles = p.tiles
        cur = self.tile_args(tiles[ti])
        nxt = self.tile_args(tiles[ti + 1] if ti + 1 < len(tiles) else tiles[ti])
        S, V = self.S, self.V
        for k, v in (("A", cur["A"]), ("B", cur["B"]), ("An", nxt["A"]), ("Bn", nxt["B"]), ("mxa", cur["mxa"]), ("mxb", cur["mxb"]),
                     ("mxan", nxt["mxa"]), ("mxbn", nxt["mxb"]), ("wl", LDS0 + self.wave * 1024),
                     ("kh", ((tiles[ti][3] - tiles[ti][2]) if len(tiles[ti]) > 2 else p.ksteps) // 2), ("first", first), ("nst", nst), ("fe", fe), ("cprev", cprev),
                     ("cstep", p.C.stride * 16), ("scbuf", scbuf)):
            S[f"%[{k}]"] = v
        m0, n0 = tiles[ti][:2]
        whole = m0 + 256 <= p.m and n0 + 256 <= p.n
        regs = p.scaled and whole
        S["%[sap]"] = p.sa.base + 4 * (m0 + self.wm0) if regs else cur["A"]
        S["%[sbp]"] = p.sb.base + 4 * (n0 + self.wn0) if regs else cur["B"]
        for i in range(16):
            V[192 + i] = cur["off"][i] & MASK32
            V[208 + i] = nxt["off"][i] & MASK32
        m = (self.r & 7) ^ (self.r >> 3)
        lo = ((2 * self.g) ^ m) << 4
        a0 = LDS0 + (self.wm0 + self.r) * 128 + lo
        b0 = LDS0 + 32768 + (self.wn0 + self.r) * 128 + lo
        for i, v in enumerate((a0, a0 ^ 16, b0, b0 ^ 16, a0 + 65536, (a0 ^ 16) + 65536, b0 + 65536, (b0 ^ 16) + 65536)):
            V[224 + i] = v
        coff = (self.r * p.C.stride + 16 * self.g) & MASK32      # ((r * c_sm + 8 g) * 2 with c_sm in elements)
        if p.fp4:
            V[232] = LDS0 + SC0 + (self.wm0 + self.r) * 16 + self.g * 2
            V[233] = LDS0 + SC0 + (256 + self.wn0 + self.r) * 16 + self.g * 2
            V[234], V[235], V[236], V[237] = cur["sca"] & MASK32, cur["scb"] & MASK32, nxt["sca"] & MASK32, nxt["scb"] & MASK32
            V[238] = coff
        else:
            eps = g.EPS
            V[240] = coff
            V[241] = self.lane * 4
            V[242] = LDS0 + eps + self.wave * 1024 + self.r * 4
            V[243] = LDS0 + eps + self.wave * 1024 + 512 + self.g * 32

    # ---- values ---------------------------------------------------------------------------------------------------
    def sval(self, tok, bits=32):
        tok = tok.strip()
        m = re.fullmatch(r"s\[(\d+):(\d+)\]", tok)
        if m:
            return self.S[f"s{m.group(1)}"] | (self.S[f"s{m.group(2)}"] << 32)
        if tok in self.S:
            return self.S[tok]
        if re.fullmatch(r"-?\d+", tok):
            return int(tok) & (MASK64 if bits == 64 else MASK32)
        raise Fail(f"unknown scalar operand {tok}")

    def sset(self, tok, val, bits=32):
        tok = tok.strip()
        m = re.fullmatch(r"s\[(\d+):(\d+)\]", tok)
        if m:
            self.S[f"s{m.group(1)}"], self.S[f"s{m.group(2)}"] = val & MASK32, (val >> 32) & MASK32
        elif tok.startswith("%["):
            self.S[tok] = val & MASK32              # (an in/out operand of the statement)
        else:
            self.S[tok] = val & MASK32

    def vval(self, tok):
        tok = tok.strip()
        m = re.fullmatch(r"v(\d+)", tok)
        if m:
            n = int(m.group(1))
            if n not in self.V:
                raise Fail(f"address register v{n} was never written")
            return self.V[n]
        return np.full(64, self.sval(tok), dtype=np.int64)

    # ---- memory operations -----------------------------------------------------------------------------------------
    def lds_area(self, off):
        """name of the LDS area byte offset `off` (relative to the array) belongs to"""
        g = self.gen
        if 0 <= off < 2 * STAGE:
            return ("A", "B")[(off % STAGE) // BOFF] + str(off // STAGE)
        top = SC0 + 16384
        if self.prob.fp4 and SC0 <= off < top:
            return "scale"
        if not self.prob.fp4 and g.EPS <= off < g.EPS + 4096:
            return "eps"
        raise Fail(f"LDS offset {off} is in no area of this kernel")

    def copy(self, vreg, base, size):
        """LDS-direct load: lane l fetches `size` bytes at base + v[l] and writes them at m0 + l * size"""
        voff = self.vval(vreg)
        m0 = self.S["m0"] - LDS0
        entry = {"done": False, "lds": []}
        self.vmq.append(entry)
        allowed = {"A": ("A",), "B": ("B",), "scale": ("mxa", "mxb"),
                   # (a tile without scale vectors copies 512 bytes of its operands there instead; nobody reads them)
                   "eps": ("sa", "sb", "A", "B")}
        for l in range(64):
            addr = base + int(voff[l])
            where = None
            for sp in self.prob.spaces:
                loc = sp.locate(addr, size)
                if loc is not None:
                    where = (sp.name,) + loc
            if where is None:
                raise Fail(f"copy {vreg} lane {l}: [{addr:#x}, +{size}) is outside every operand (step {self.step})")
            off = m0 + l * size
            area = self.lds_area(off)
            if where[0] not in allowed[area.rstrip("01")]:
                raise Fail(f"copy of {where[0]} goes to LDS area {area}")
            for b in range(0, size, 4):
                o = off + b
                # write after read: the last read of these bytes must have completed before the latest barrier
                if any(w.last_read.get(o, 0) > w.covered for w in self.group.waves):
                    raise Fail(f"copy overwrites LDS {o} ({area}) whose last read had not completed at the latest barrier (step {self.step})")
                self.lds[o] = {"what": (where[0], where[1], where[2] + b), "vm": entry, "pub": False}
                entry["lds"].append(o)

    def read(self, dst, areg, imm, size):
        addr = self.vval(areg) + imm - LDS0
        self.reads += 1
        self.outstanding += 1
        out = []
        for l in range(64):
            lane = []
            for b in range(0, max(size, 4), 4):
                o = (int(addr[l]) + b) & ~3
                self.lds_area(o)
                e = self.lds.get(o)
                if e is None:
                    raise Fail(f"LDS read of {o} ({self.lds_area(o)}): nothing was ever copied there (step {self.step})")
                if not e["pub"]:
                    raise Fail(f"LDS read of {o} ({self.lds_area(o)}) before its copy was awaited and published by a barrier (step {self.step}, {e['what']})")
                self.last_read[o] = self.reads
                lane.append(e["what"])
            out.append((lane, int(addr[l]) & 3))
        return out

    # ---- what a fragment read must have fetched -----------------------------------------------------------------------
    def expect_rows(self, space, t, tile):
        m0, n0 = self.prob.tiles[tile][:2]
        if space in ("A", "mxa"):
            return np.minimum(m0 + self.wm0 + 16 * t + self.r, self.prob.m - 1)
        rows = np.array([b_tile_row(int(x)) for x in (self.wn0 + 16 * t + self.r)])
        return np.minimum(n0 + rows, self.prob.n - 1)

    def note_fragment(self, dst, got):
        """ds_read_b128 of half a fragment: which operand, K step and half the lanes agree on, and each lane's row"""
        keys = set()
        for l in range(64):
            lane, _ = got[l]
            sp, row, col = lane[0]
            if any(x != (sp, row, col + 4 * i) for i, x in enumerate(lane)):
                raise Fail("a 16-byte fragment read spans two copies")
            kstep, c = divmod(col, 128)
            if c % 16:
                raise Fail("misaligned fragment chunk")
            c //= 16
            if c >> 1 != self.g[l]:
                raise Fail(f"lane {l} of a fragment read got chunk {c}, expected {2 * self.g[l]} or {2 * self.g[l] + 1}")
            keys.add((sp, kstep, c & 1))
        if len(keys) != 1:
            raise Fail(f"lanes of a fragment read disagree: {keys}")
        sp, kstep, half = keys.pop()
        rows = np.array([got[l][0][0][1] for l in range(64)])
        for r in self.gen.Gen._vregs(dst):
            self.meta[r] = ("frag", sp, kstep, half, rows)

    def note_scale(self, dst, got):
        regs = self.gen.Gen._vregs(dst)
        info = []
        for l in range(64):
            lane, sub = got[l]
            sp, row, col = lane[0]
            info.append((sp, row, col + sub))
        for r in regs:
            self.meta[r] = ("scale", info)

    def mfma(self, text):
        m = re.match(r"v_mfma\S+ a\[(\d+):\d+\], v\[(\d+):(\d+)\], v\[(\d+):(\d+)\], (\S+?),?( v(\d+), v(\d+) op_sel:\[(\d),(\d),0\])?( |$)", text)
        if not m:
            raise Fail(f"cannot parse {text}")
        acc = int(m.group(1)) // 4
        i, j = acc // 8, acc % 8
        tile, kstep = self.step
        for first, last, space, t in ((int(m.group(2)), int(m.group(3)), "B", j), (int(m.group(4)), int(m.group(5)), "A", i)):
            want_rows = self.expect_rows(space, t, tile)
            for r in range(first, last + 1):
                md = self.meta.get(r)
                if md is None or md[0] != "frag":
                    raise Fail(f"{text}: v{r} holds no fragment")
                _, sp, ks, hf, rows = md
                if sp != space or ks != kstep or not np.array_equal(rows, want_rows):
                    raise Fail(f"MFMA for accumulator ({i}, {j}) of tile {tile} step {kstep} reads v{r} = {sp} step {ks} rows {rows[:3]}.. (wanted {space} rows {want_rows[:3]}..)")
            if last - first == 7:
                # FP8: both halves in one instruction, low registers = chunk 2g
                if [self.meta[first][3], self.meta[first + 4][3]] != [0, 1]:
                    raise Fail(f"{text}: halves of a fragment in the wrong registers")
        if m.group(7):
            # MXFP4: the E8M0 byte of this lane's row and K block (lane group g owns blocks 2g, 2g+1 of a K step)
            ks_sel = int(m.group(10))
            if int(m.group(11)) != ks_sel:
                raise Fail("op_sel of the two scales differ")
            a_half = self.meta[int(m.group(4))][3]
            if a_half != ks_sel or self.meta[int(m.group(2))][3] != ks_sel:
                raise Fail(f"{text}: k slice {ks_sel} multiplies half {a_half}")
            for reg, space, t in ((int(m.group(8)), "mxb", j), (int(m.group(9)), "mxa", i)):
                md = self.meta.get(reg)
                if md is None or md[0] != "scale":
                    raise Fail(f"{text}: v{reg} holds no scales")
                want_rows = self.expect_rows(space, t, tile)
                for l in range(64):
                    sp, row, col = md[1][l]
                    if sp != space or row != want_rows[l] or col != kstep * 8 + 2 * int(self.g[l]):
                        raise Fail(f"{text}: lane {l} scale register v{reg} holds {sp} row {row} byte {col}, wanted {space} row {want_rows[l]} byte {kstep * 8 + 2 * int(self.g[l])}")
        elif self.prob.fp4:
            raise Fail("unscaled MFMA in an MXFP4 loop")
        else:
            # 16-bit / int8 kinds: two MFMAs per accumulator and K step, half h of A with half h of B
            if int(m.group(3)) - int(m.group(2)) == 3 and self.meta[int(m.group(2))][3] != self.meta[int(m.group(4))][3]:
                raise Fail(f"{text}: halves of A and B differ")

    def wait_vm(self, n):
        done = len(self.vmq) - n
        for e in self.vmq[:max(0, done)]:
            e["done"] = True

    def barrier(self):
        """this wave's part of a barrier (all four waves are at the same instruction)"""
        for e in self.vmq:
            if e["done"]:
                for o in e["lds"]:
                    if self.lds.get(o, {}).get("vm") is e:
                        self.lds[o]["pub"] = True
        self.vmq = [e for e in self.vmq if not e["done"]]
        self.covered = self.reads - self.outstanding

    def store(self, text, prev_tile):
        m = re.match(r"global_store_dwordx4 v(\d+), v\[\d+:\d+\], (s\[\d+:\d+\]) offset:(\d+)", text)
        base = self.sval(m.group(2)) + int(m.group(3))
        voff = self.vval("v" + m.group(1))
        self.vmq.append({"done": False, "lds": []})
        p = self.prob
        m0, n0 = p.tiles[prev_tile][:2]
        for l in range(64):
            addr = base + int(voff[l])
            loc = p.C.locate(addr, 16)
            if loc is None:
                raise Fail(f"store outside C: {addr:#x}")
            row, col = loc
            if not (m0 + self.wm0 <= row < m0 + self.wm0 + 128 and 2 * (n0 + self.wn0) <= col < 2 * (n0 + self.wn0 + 128)):
                raise Fail(f"store of the fused epilogue outside the wave's quarter of the previous tile: row {row} byte {col}")
            self.stores[addr] = self.stores.get(addr, 0) + 1

    # ---- the interpreter -----------------------------------------------------------------------------------------------
    def execute(self, t, op, rest, a, tile, prev_tile):
        """one instruction that is not a branch"""
        S = self.S
        if op == "s_mov_b32":
            self.sset(a[0], self.sval(a[1]))
        elif op == "s_mov_b64":
            self.sset(a[0], self.sval(a[1], 64), 64)
        elif op in ("s_add_u32", "s_addc_u32", "s_sub_u32", "s_subb_u32"):
            x, y = self.sval(a[1]), self.sval(a[2])
            c = S.get("scc", 0)
            if op == "s_add_u32":
                v = x + y
            elif op == "s_addc_u32":
                v = x + y + c
            elif op == "s_sub_u32":
                v = x - y
            else:
                v = x - y - c
            S["scc"] = 1 if (v > MASK32 or v < 0) else 0
            self.sset(a[0], v & MASK32)
        elif op in ("s_xor_b32", "s_and_b32"):
            x, y = self.sval(a[1]), self.sval(a[2])
            self.sset(a[0], (x ^ y) if op == "s_xor_b32" else (x & y))
        elif op == "s_xor_b64":
            self.sset(a[0], self.sval(a[1], 64) ^ self.sval(a[2], 64), 64)
        elif op in ("s_cmp_eq_u32", "s_cmp_lg_u32"):
            eq = self.sval(a[0]) == self.sval(a[1])
            S["scc"] = int(eq if op == "s_cmp_eq_u32" else not eq)
        elif op == "s_nop":
            pass
        elif op == "s_barrier":
            self.barrier()
        elif op == "s_waitcnt":
            n = int(rest[rest.index("(") + 1:rest.index(")")])
            if rest.startswith("vmcnt"):
                self.wait_vm(n)
            else:
                self.outstanding = min(self.outstanding, n)
        elif op in ("v_mov_b32", "v_xor_b32", "v_add_u32"):
            d = int(a[0][1:])
            if op == "v_mov_b32":
                self.V[d] = self.vval(a[1]).copy()
            elif op == "v_xor_b32":
                self.V[d] = (self.vval(a[1]) ^ self.vval(a[2])) & MASK32
            else:
                self.V[d] = (self.vval(a[1]) + self.vval(a[2])) & MASK32
            self.meta.pop(d, None)
        elif op.startswith("global_load_lds"):
            self.copy(a[0], self.sval(a[1], 64), 16 if op.endswith("dwordx4") else 4)
        elif op.startswith("ds_read"):
            areg, _, tail = a[1].partition(" ")
            imm = int(tail.split("offset:")[1]) if "offset:" in tail else 0
            size = {"ds_read_b128": 16, "ds_read_b32": 4, "ds_read_u16": 2}[op]
            got = self.read(a[0], areg, imm, size)
            area = self.lds_area(int(self.vval(areg)[0]) + imm - LDS0)
            for r in self.gen.Gen._vregs(a[0]):
                self.meta.pop(r, None)
            if area[0] in "AB" and size == 16:
                self.note_fragment(a[0], got)
            elif area == "scale":
                self.note_scale(a[0], got)
            else:
                self.note_eps(a[0], got, prev_tile)
        elif op.startswith("v_mfma"):
            self.mfma(t)
        elif op.startswith("global_store"):
            self.store(t, prev_tile)
        elif op.startswith("v_"):
            # arithmetic of the fused epilogue: the destination no longer holds what an LDS read put there
            m = re.fullmatch(r"v(\d+)", a[0]) if a else None
            if m:
                self.meta.pop(int(m.group(1)), None)
                if int(m.group(1)) in self.V and int(m.group(1)) >= 192:
                    raise Fail(f"{t} overwrites an address register")
        else:
            raise Fail(f"instruction the replay does not know: {t}")

    def note_eps(self, dst, got, prev_tile):
        """epilogue scales read back: the wave's rows 16 i + r of sa and columns 32 q + 8 g + 4 h + 0..3 of sb of the PREVIOUS tile"""
        p = self.prob
        m0, n0 = p.tiles[prev_tile][:2]
        regs = sorted(self.gen.Gen._vregs(dst))
        for l in range(64):
            lane, _ = got[l]
            for k, (sp, row, col) in enumerate(lane):
                idx = col // 4
                if sp == "sa":
                    i = (regs[0] - 96)
                    want = m0 + self.wm0 + 16 * i + int(self.r[l])
                elif sp == "sb":
                    base = regs[0] - 64          # 8 q + 4 h
                    want = n0 + self.wn0 + 32 * (base // 8) + 8 * int(self.g[l]) + 4 * ((base // 4) % 2) + k
                else:
                    raise Fail(f"epilogue scale read got {sp}")
                if idx != want:
                    raise Fail(f"epilogue scale register v{regs[0] + (k if sp == 'sb' else 0)} lane {l}: {sp}[{idx}], wanted [{want}]")


class Group:
    """the four waves of a workgroup, in step through one statement"""
    def __init__(self, gen, prob):
        self.lds = {}
        self.waves = []
        for wv in range(4):
            self.waves.append(Wave(gen, prob, wv, self))

    def run(self, lines, tile, prev_tile, first_step=0):
        labels = {l[:-1]: n for n, l in enumerate(lines) if l.endswith(":")}
        pc, kstep = 0, None
        while pc < len(lines):
            t = lines[pc]
            pc += 1
            if t.endswith(":"):
                continue
            if t.startswith(";"):
                if "K step" in t:
                    kstep = first_step if kstep is None else kstep + 1
                    for w in self.waves:
                        w.step = (tile, kstep)
                continue
            op, _, rest = t.partition(" ")
            a = [x.strip() for x in rest.split(",")] if rest else []
            if op in ("s_cbranch_scc1", "s_cbranch_scc0", "s_branch"):
                scc = {w.S.get("scc", 0) for w in self.waves}
                if len(scc) != 1:
                    raise Fail(f"{t}: the waves of a workgroup disagree")
                if op == "s_branch" or scc.pop() == (1 if op.endswith("1") else 0):
                    pc = labels[a[0]]
                continue
            for w in self.waves:
                w.execute(t, op, rest, a, tile, prev_tile)


def replay(kind, m, n, ksteps, tiles, c_bf16=True, pad=0, env=None):
    """Runs the generated program of `kind` over `tiles` (list of (m0, n0), or (m0, n0, it0, it1) for a Stream-K
    piece that covers K steps [it0, it1) of its tile) for the four waves of a workgroup, the
    way the loop of gemm_kernel_w4 would (history flags, fused or compiled epilogues).  Raises Fail on the first
    violation; returns the number of MFMAs checked."""
    gen = load_generator()
    old = {}
    for k, v in (env or {}).items():
        old[k] = os.environ.get(k)
        os.environ[k] = v
    try:
        g = gen.Gen(kind)
        lines = [l.replace("%=", "") for l in g.program()]
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    prob = Problem(kind, m, n, ksteps, tiles, pad=pad)
    grp = Group(gen, prob)
    checked = 0
    first, nst, fe, scbuf = 1, 0, 0, 0
    cprev = [prob.C.base] * 4
    for ti, item in enumerate(tiles):
        m0, n0 = item[:2]
        piece = len(item) > 2          # a Stream-K piece (K steps [it0, it1)): its sums leave through compiled code
        have_next = ti + 1 < len(tiles)
        whole = m0 + 256 <= m and n0 + 256 <= n
        fast = whole and not piece
        fe_shape = c_bf16
        before = []
        for w in grp.waves:
            w.bind(ti, first, nst, fe, cprev[w.wave], scbuf)
            before.append(dict(w.stores))
        grp.run(lines, ti, ti - 1, item[2] if piece else 0)
        checked += 4 * ((item[3] - item[2]) if piece else ksteps) * (64 if kind in ("fp8", "e5m2") else 128)
        scbuf = grp.waves[0].S["%[scbuf]"]
        for w in grp.waves:
            if fe:
                # the wave's quarter of the previous tile: every 16 bytes exactly once
                pm, pn = tiles[ti - 1][:2]
                for row in range(pm + w.wm0, pm + w.wm0 + 128):
                    for col in range(2 * (pn + w.wn0), 2 * (pn + w.wn0 + 128), 16):
                        a = prob.C.base + row * prob.C.stride + col
                        if w.stores.get(a, 0) - before[w.wave].get(a, 0) != 1:
                            raise Fail(f"fused epilogue wrote C row {row} byte {col} {w.stores.get(a, 0) - before[w.wave].get(a, 0)} times")
            cprev[w.wave] = prob.C.base + (m0 + w.wm0) * prob.C.stride + (n0 + w.wn0) * 2
            if not (fast and fe_shape and have_next):
                for _ in range(32 if fast else w.ragged_stores):
                    w.vmq.append({"done": False, "lds": []})
        if fast and fe_shape and have_next:
            fe, nst = 1, 0
        else:
            fe, nst = 0, (1 if fast else 0)
        first = 0
    return checked
