"""Generator of the hand-scheduled k-loop of the bf16 contraction kernels (gfx950).

Writes ``mainloop16.inc``: for each operand-layout variant, the assembly text of the loop over
the k-tiles of one 256 x 256 output tile, as C string macros that ``lmhead.hip`` places in an
``asm volatile`` statement.  The loop is emitted instruction by instruction so that the issue
order is the one written here, whatever the compiler would have scheduled:

* the MFMA is ``v_mfma_f32_16x16x32_bf16`` with all 64 accumulator blocks of a wave in
  ``a[0:255]``: block (ia, jb) of the wave's 128 x 128 sub-tile in ``a[(8 ia + jb) * 4 ..+3]``;
* a k-tile (64 k) is two k-steps of 64 MFMAs.  The A fragments of a k-step live in one of two
  register buffers and are fetched from LDS during the k-step before; the B fragments of a whole
  k-tile (both k-steps) are fetched during the second k-step of the k-tile before, into one of
  two pairs of buffers;
* operands travel global -> LDS directly (``global_load_lds_dwordx4``) into a ring of two
  stages.  Because a k-tile's B fragments leave LDS a k-step earlier than its A fragments, the B
  half of a stage is refilled from the start of the k-tile that consumes the stage and the A
  half from its middle: two half-batches of loads are in flight at any time and each has a full
  k-tile (the B half one and a half) to land, so the load pipe never drains.  One barrier at the
  start and one in the middle of a k-tile publish a landed half and retire a consumed one.  The
  8 loads of a half-batch are issued several MFMAs apart (``LOAD_SPACING``), not back to back;
* two k-tiles (one per stage) form the loop body, and the LDS is laid out as
  ``[A stage 0][A stage 1][B stage 0][B stage 1]`` (32 KB each) so that the two stages of an
  operand differ by an immediate offset: every LDS address is one register plus an immediate
  and the loop spends no vector instruction on addresses.

Operand layouts: ``kc`` = k contiguous (row = i or j, 128 B of k per stage row, 16-byte chunks
XOR-swizzled), ``km`` = k major (row = k, 512 B of i or j per stage row, fetched with
``ds_read_b64_tr_b16``).  Variants: nt = (kc, kc), tn = (km, km), mix = (km, kc).

An odd number of k-tiles runs as one more pair whose second k-tile is "dead": it keeps the
pipeline's loads, fragment reads and barriers (the next output tile's first two k-tiles arrive in
the same stages as always) and issues no MFMA.  The loads that would fetch the k-tile behind the
last one are issued with the pointers held back by one k-tile (``S_PEN_*`` replaces the stride
for one advance), so they fetch the last k-tile again and nothing outside the operands is read.

Run ``python gen_mainloop16.py`` to rewrite ``mainloop16.inc`` next to this file.
"""

from __future__ import annotations

import sys
from pathlib import Path

# ---- physical registers of the asm block (the C++ side binds its operands to the same names)
S_PA, S_PB, S_PA_NEXT, S_PB_NEXT = 40, 42, 44, 46  # 64-bit pointers: s[n:n+1]
S_CNT, S_LDSW, S_STRIDE_A, S_STRIDE_B = 48, 49, 50, 51
# odd k-tile counts: S_ODD = 1 when the tile's last pair has a dead second k-tile (else 0);
# S_PEN_* = what the pointers advance by after the loads of the tile's last real k-tile
# (0 for an odd count, the stride otherwise); S_EFF_* are scratch
S_ODD, S_PEN_A, S_PEN_B, S_EFF_A, S_EFF_B = 52, 53, 54, 55, 56

HALF_BYTES = 32768            # one operand of one stage
OPER_BYTES = 2 * HALF_BYTES   # both stages of one operand


class Variant:
    def __init__(self, name: str, a_km: bool, b_km: bool):
        self.name, self.km = name, (a_km, b_km)
        top = 256

        def alloc(n):
            nonlocal top
            top -= n
            return top

        # fragment buffers, 8 blocks x 4 registers each: A by k-step, B by (k-tile parity, k-step)
        self.fa = [alloc(32), alloc(32)]
        self.fb = [[alloc(32), alloc(32)], [alloc(32), alloc(32)]]
        self.off = [alloc(8), alloc(8)]  # per-lane global byte offsets of the 8 loads per half
        # LDS read address registers (stage 0; stage 1 is +HALF_BYTES): km one per block x, kc
        # one per k-step
        self.rd = [alloc(8 if self.km[o] else 2) for o in range(2)]
        self.first_vgpr = top

    # ---------------------------------------------------------------- single instructions
    def mfma(self, abuf, bbuf, ia, jb, init):
        acc = (ia * 8 + jb) * 4
        a = abuf + 4 * ia
        b = bbuf + 4 * jb
        c = "0" if init else f"a[{acc}:{acc + 3}]"
        return f"v_mfma_f32_16x16x32_bf16 a[{acc}:{acc + 3}], v[{a}:{a + 3}], v[{b}:{b + 3}], {c}"

    def reads(self, dst, stage, ks, oper, x):
        """LDS -> the 4 registers at dst: block x of operand oper, k-step ks of `stage`."""
        st = stage * HALF_BYTES
        if self.km[oper]:
            r = self.rd[oper] + x
            o = st + ks * 16384
            return [f"ds_read_b64_tr_b16 v[{dst}:{dst + 1}], v{r} offset:{o}",
                    f"ds_read_b64_tr_b16 v[{dst + 2}:{dst + 3}], v{r} offset:{o + 2048}"]
        r = self.rd[oper] + ks
        return [f"ds_read_b128 v[{dst}:{dst + 3}], v{r} offset:{st + x * 2048}"]

    def load(self, stage, oper, i):
        """(SALU that points M0 at the LDS destination, the direct load)."""
        imm = oper * OPER_BYTES + stage * HALF_BYTES + i * 1024
        ptr = S_PA if oper == 0 else S_PB
        return (f"s_add_u32 m0, s{S_LDSW}, {imm}",
                f"global_load_lds_dwordx4 v{self.off[oper] + i}, s[{ptr}:{ptr + 1}]")

    @staticmethod
    def advance(oper, eff=False):
        """Move the operand's pointer to the next k-tile; eff: by the amount select_advance() chose."""
        p, st = (S_PA, S_EFF_A if eff else S_STRIDE_A) if oper == 0 else (S_PB, S_EFF_B if eff else S_STRIDE_B)
        return [f"s_add_u32 s{p}, s{p}, s{st}", f"s_addc_u32 s{p + 1}, s{p + 1}, 0"]

    @staticmethod
    def select_advance():
        """In front of a pair: its first k-tile fetches the tile's last real k-tile exactly when
        this is the last pair but one; the pointers then advance by S_PEN_* instead of the stride."""
        return [f"s_cmp_eq_u32 s{S_CNT}, 2",
                f"s_cselect_b32 s{S_EFF_A}, s{S_PEN_A}, s{S_STRIDE_A}",
                f"s_cselect_b32 s{S_EFF_B}, s{S_PEN_B}, s{S_STRIDE_B}"]

    # ---------------------------------------------------------------- schedule
    def a_reads(self, buf, stage, ks, na=8):
        out = []
        for x in range(na):
            out += self.reads(self.fa[buf] + 4 * x, stage, ks, 0, x)
        return out

    def b_reads(self, parity, stage):
        out = []
        for ks in range(2):
            for x in range(8):
                out += self.reads(self.fb[parity][ks] + 4 * x, stage, ks, 1, x)
        return out

    def kstep(self, abuf, bbuf, init, pre, post, dead=False, na=8):
        """64 MFMA slots; pre[m] / post[m] are emitted in front of / behind slot m. dead: no MFMA;
        na < 8: the slots of the A blocks ia >= na stay empty (a narrower A tile)."""
        out = []
        for m in range(64):
            out += pre.get(m, [])
            if not dead and (m >> 3) < na:
                out.append(self.mfma(abuf, bbuf, m >> 3, m & 7, init))
            out += post.get(m, [])
        return out

    @staticmethod
    def spread(ops, first, last, into=None):
        """Place ops behind the MFMAs first..last, evenly."""
        post = {} if into is None else into
        n = len(ops)
        for r, op in enumerate(ops):
            m = first + (r * (last - first + 1)) // n
            post.setdefault(m, []).append(op)
        return post

    # MFMAs between two direct loads of a half-batch. Issued back to back (one per MFMA) the 8
    # loads of a wave congest the address path and the whole loop runs 6-8 % slower; spaced 3 to 8
    # MFMAs apart it does not matter much by how many. The B half, which has a k-tile and a half
    # to land, is spread wider than the A half, which has one k-tile.
    LOAD_SPACING = {0: 4, 1: 6}

    def put_loads(self, stage, oper, pre, post):
        step = self.LOAD_SPACING[oper]
        for i in range(8):
            setm0, ld = self.load(stage, oper, i)
            pre.setdefault(i * step, []).append(setm0)
            post.setdefault(i * step, []).append(ld)
        # the first k-tile of a pair (stage 0) advances by the selected amount
        post.setdefault(7 * step + 1, []).extend(self.advance(oper, eff=(stage == 0)))

    def ktile(self, parity, init, dead=False, na=8):
        stage = parity
        barrier = ["s_barrier"]
        out = [f"; ---- k-tile on stage {stage}{' (dead: no MFMA)' if dead else ''}: k-step 0"]
        # k-step 0: the B half of this stage is free (its fragments are in registers): refill
        # it with the k-tile after next; A fragments of k-step 1 -> A buffer 1
        pre, post = {}, {}
        self.put_loads(stage, 1, pre, post)
        self.spread(self.a_reads(1, stage, 1, na), 9, 40, post)
        out += self.kstep(self.fa[0], self.fb[parity][0], init, pre, post, dead, na)
        # own A reads done and own loads of one k-tile ago landed (the 8 newest may be in flight)
        out += ["s_waitcnt vmcnt(8) lgkmcnt(0)"] + barrier
        out += [f"; ---- k-tile on stage {stage}: k-step 1"]
        # k-step 1: the A half of this stage is free: refill it; from the other stage (landed,
        # published by the barrier) A fragments of k-step 0 -> A buffer 0 and all B fragments
        # of the next k-tile -> the other pair of B buffers
        pre, post = {}, {}
        self.put_loads(stage, 0, pre, post)
        # the last fragment read sits 11 MFMAs in front of the k-step's end, whatever its length
        self.spread(self.a_reads(0, stage ^ 1, 0, na) + self.b_reads(parity ^ 1, stage ^ 1), 9, 8 * na - 12, post)
        out += self.kstep(self.fa[1], self.fb[parity][1], False, pre, post, dead, na)
        # every wave has the next k-tile's B fragments: the other stage's B half may be refilled
        out += ["s_waitcnt lgkmcnt(0)"] + barrier
        return out

    def pair(self, init, dead_second=False, na=8):
        return self.select_advance() + self.ktile(0, init, False, na) + self.ktile(1, False, dead_second, na)

    def tile_loop(self, na=8):
        """One 256 x 256 tile: s48 pairs of k-tiles, the second k-tile of the last pair dead when
        s52 is 1 (an odd number of k-tiles; then at least two pairs). On entry both stages hold (or
        are receiving) k-tiles 0 and 1 and the pointers are on the next k-tile to fetch.
        na < 8: a tile of 32 na x 256, each wave's sub-tile 16 na x 128: the loads, barriers and B
        fragment reads are those of the full tile; the fragment reads and MFMAs of the A blocks
        ia >= na are left out."""
        out = ["s_waitcnt vmcnt(0) lgkmcnt(0)", "s_barrier"]
        out += self.a_reads(0, 0, 0, na) + self.b_reads(0, 0)
        out += ["s_waitcnt lgkmcnt(0)", "s_barrier"]
        out += self.pair(True, False, na)
        out += [f"s_sub_u32 s{S_CNT}, s{S_CNT}, 1", f"s_cmp_eq_u32 s{S_CNT}, 0", "s_cbranch_scc1 2f", "1:",
                # the last pair fetches the next tile's first k-tiles
                f"s_cmp_eq_u32 s{S_CNT}, 1",
                f"s_cselect_b64 s[{S_PA}:{S_PA + 1}], s[{S_PA_NEXT}:{S_PA_NEXT + 1}], s[{S_PA}:{S_PA + 1}]",
                f"s_cselect_b64 s[{S_PB}:{S_PB + 1}], s[{S_PB_NEXT}:{S_PB_NEXT + 1}], s[{S_PB}:{S_PB + 1}]",
                # ... and is the one with the dead k-tile if the count is odd (s52 = 1; 0 never matches)
                f"s_cmp_eq_u32 s{S_CNT}, s{S_ODD}", "s_cbranch_scc1 3f"]
        out += self.pair(False, False, na)
        out += [f"s_sub_u32 s{S_CNT}, s{S_CNT}, 1", f"s_cmp_lg_u32 s{S_CNT}, 0", "s_cbranch_scc1 1b",
                "s_branch 2f", "3:"]
        out += self.pair(False, True, na)
        out += ["2:", "s_nop 15", "s_nop 15"]  # the last MFMAs retire before the accumulators are read
        return out

    def prologue(self):
        """k-tiles 0 and 1 of the first tile -> stages 0 and 1."""
        out = []
        for stage in (0, 1):
            for oper in (0, 1):
                for i in range(8):
                    setm0, ld = self.load(stage, oper, i)
                    out += [setm0, "s_nop 0", ld]
            out += self.advance(0) + self.advance(1)
        return out

    def clobbers(self):
        lo = self.fb[1][1]
        return [f"v{r}" for r in range(lo, 256)]


def cstring(lines):
    return " \\\n".join('  "' + ln + '\\n\\t"' for ln in lines)


def emit():
    variants = [Variant("NT", False, False), Variant("TN", True, True), Variant("MIX", True, False)]
    out = ["// Generated by gen_mainloop16.py: do not edit.", "#pragma once", ""]
    out += [f"#define ML16_S_PA \"{{s[{S_PA}:{S_PA + 1}]}}\"", f"#define ML16_S_PB \"{{s[{S_PB}:{S_PB + 1}]}}\"",
            f"#define ML16_S_PA_NEXT \"{{s[{S_PA_NEXT}:{S_PA_NEXT + 1}]}}\"",
            f"#define ML16_S_PB_NEXT \"{{s[{S_PB_NEXT}:{S_PB_NEXT + 1}]}}\"",
            f"#define ML16_S_CNT \"{{s{S_CNT}}}\"", f"#define ML16_S_LDSW \"{{s{S_LDSW}}}\"",
            f"#define ML16_S_STRIDE_A \"{{s{S_STRIDE_A}}}\"", f"#define ML16_S_STRIDE_B \"{{s{S_STRIDE_B}}}\"",
            f"#define ML16_S_ODD \"{{s{S_ODD}}}\"", f"#define ML16_S_PEN_A \"{{s{S_PEN_A}}}\"",
            f"#define ML16_S_PEN_B \"{{s{S_PEN_B}}}\"",
            f"#define ML16_S_SCRATCH_CLOBBERS \"s{S_EFF_A}\", \"s{S_EFF_B}\"",
            f"#define ML16_HALF_BYTES {HALF_BYTES}", f"#define ML16_OPER_BYTES {OPER_BYTES}", ""]
    # The accumulators are not operands: the compiler must not know values live in a[0:255]
    # (it would move them around); the main loop lists them as clobbered.
    out.append("#define ML16_ACC_CLOBBERS " + ", ".join(f'"a{i}"' for i in range(256)))
    # Block column jb of a wave's accumulators (8 blocks ia x 4 registers) to 32 VGPRs:
    # x[ia * 4 + r] = a[(ia * 2 + jb / 4) * 16 + (jb % 4) * 4 + r]
    out.append("#define ML16_COL_OUTPUTS(x) " + ", ".join(f'"=v"(x[{i}])' for i in range(32)))
    for jb in range(8):
        lines = [f"v_accvgpr_read_b32 %{ia * 4 + r}, a{(ia * 2 + jb // 4) * 16 + (jb % 4) * 4 + r}"
                 for ia in range(8) for r in range(4)]
        out.append(f"#define ML16_READ_COL{jb} \\\n" + cstring(lines))
    out.append("")
    for v in variants:
        n = v.name
        out.append(f"// ---- {n}: A {'k-major' if v.km[0] else 'k-contiguous'}, "
                   f"B {'k-major' if v.km[1] else 'k-contiguous'}; asm block uses v[{v.first_vgpr}:255]")
        out.append(f"#define ML16_{n}_FIRST_VGPR {v.first_vgpr}")
        ins = [f'"{{v{v.off[0] + i}}}"(oa[{i}])' for i in range(8)]
        ins += [f'"{{v{v.off[1] + i}}}"(ob[{i}])' for i in range(8)]
        ins += [f'"{{v{v.rd[0] + i}}}"(ra[{i}])' for i in range(8 if v.km[0] else 2)]
        ins += [f'"{{v{v.rd[1] + i}}}"(rb[{i}])' for i in range(8 if v.km[1] else 2)]
        out.append(f"#define ML16_{n}_VGPR_INPUTS(oa, ob, ra, rb) " + ", ".join(ins))
        out.append(f"#define ML16_{n}_CLOBBERS " + ", ".join(f'"{c}"' for c in v.clobbers()))
        out.append(f"#define ML16_{n}_PROLOGUE \\\n" + cstring(v.prologue()))
        out.append(f"#define ML16_{n}_TILE \\\n" + cstring(v.tile_loop()))
        if v.km[0]:  # narrower A tiles exist for a k-major A (its tile column is a lane offset)
            out.append(f"#define ML16_{n}_TILE7 \\\n" + cstring(v.tile_loop(7)))
        out.append("")
    return "\n".join(out) + "\n"


if __name__ == "__main__":
    path = Path(__file__).resolve().parent / "mainloop16.inc"
    path.write_text(emit())
    print(f"wrote {path}", file=sys.stderr)
