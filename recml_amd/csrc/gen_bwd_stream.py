#!/usr/bin/env python3
"""Writes the hand-scheduled instruction stream of the dK/dV backward kernel's interior blocks.

The dK/dV kernel (hstu_attn.hip, hstu_bwd_dkv_mfma at d = 128) gives each wave 32 keys, whose K and V
fragments stay in registers, and streams tiles of 32 query rows (Q and dO) through an LDS ring.  One block is
32 matrix instructions -- S = Q K^T (8), dP = dO V^T (8), dV^T += dO^T P (8), dK^T += Q^T dS (8) -- and 176
vector instructions per lane for the 16 logits it holds (scale, exp2, add, rcp, the SiLU's derivative, two
products, the rounding of P and dS to bf16).  Written as C++ the compiler runs the phases one after the other,
and the wave, which has its SIMD to itself (the kernel needs more than 256 registers), waits out every latency.
This generator emits two consecutive blocks (t, t + 1: the pair between two of the kernel's barriers) as ONE
instruction stream in which the vector instructions of one block run behind the matrix instructions of the other:

  slots  0.. 7   S(t)
  slots  8..15   dP(t)           | vector part of block t from slot 8 on (its products with dP(t) come late enough)
  slots 16..31   S(t+1), dP(t+1) |
  slots 32..47   dV, dK (t)      | vector part of block t + 1, rows 0..15 first (slot 48 needs them)
  slots 48..55   dV, dK (t+1), rows 0..15
  slots 56..63   dV, dK (t+1), rows 16..31

Every matrix instruction takes its A operand from LDS (one 128-bit row read, or two transposing 64-bit reads),
asked for LEAD slots ahead into NRING fragment registers used in turn; waits for LDS are counted by hand, and so
are the wait states the hardware does not interlock (the emitter tracks who wrote each register and pads):

  matrix instruction (8 passes) -> vector read of its result      11
  vector write -> matrix instruction read                          2
  exp2 / rcp result -> other vector instruction                    1

Registers.  The eight accumulators (dV, dK: 128 registers) are operands in ordinary vector registers: as the C / D
operand of this matrix instruction an accumulation register was measured at about 140 cycles an instruction
against 32 (the same 32 instructions of a pair: 1.10 ms of a 1.85 ms kernel with accumulation registers, 0.23 ms
with vector registers).  The K and V fragments, B operands only, are operands in accumulation registers, which
costs nothing measurable.  The stream's own window is v[136:255]: fragments in turn (24), S and dP of both blocks
(64; the scaled logits overwrite S, and P and dS of eight rows overwrite the dP of those rows once it has been
read), temporaries of eight logits (24), eight LDS addresses (the row reads' first, the transposing reads' after
the pair's last row read).

Only blocks that need no mask and no bias qualify; the kernel keeps the compiler's code for the rest.  The
arithmetic is instruction for instruction the compiler's, in the same order per accumulator: both ways give the
same bits (tests/test_gpu_stream.py).

Usage:  python gen_bwd_stream.py [--out hstu_bwd_stream_d128.inc]
The output is C++ source: `asm volatile(...)` statements for the kernel to #include, one per variant
(HSTU_BWD_STREAM_VARIANT selects which the including code expands).
"""

from __future__ import annotations

import argparse
import os

D = 128
STAGE = 16384          # bytes of one ring stage: Q tile (8 KB) then dO tile (8 KB)
Q_BYTES = 8192
LEAD = 4               # slots between asking for a fragment and the matrix instruction that reads it
NRING = 6              # fragment registers in turn (the one asked for now was last read two slots ago)
LN2_BITS = "0x3f317218"


class Emitter:
  """Collects instructions; counts LDS reads in flight and the wait states between dependent instructions."""

  MFMA_TO_VALU = 12      # instructions (or wait states) from a matrix instruction to a vector read of its result
  VALU_TO_MFMA = 3
  TRANS_TO_VALU = 2

  def __init__(self):
    self.lines = []
    self.now = 0                   # wait states issued so far
    self.w_mfma, self.w_valu, self.w_trans = {}, {}, {}
    self.lds_issued = 0
    self.lds_done = 0
    self.tag_index = {}
    self.pads = 0

  def _raw(self, s, states=1):
    self.lines.append(s)
    self.now += states

  def _pad_to(self, when):
    """Wait states until `now` >= when."""
    while self.now < when:
      n = min(when - self.now, 8)
      self._raw(f"s_nop {n - 1}", n)
      self.pads += n

  def valu(self, text, reads=(), writes=(), trans=False):
    need = 0
    for r in reads:
      if r in self.w_mfma: need = max(need, self.w_mfma[r] + self.MFMA_TO_VALU)
      if r in self.w_trans: need = max(need, self.w_trans[r] + self.TRANS_TO_VALU)
    for r in writes:      # a vector write over a matrix result still in flight
      if r in self.w_mfma: need = max(need, self.w_mfma[r] + self.MFMA_TO_VALU)
    self._pad_to(need)
    for r in writes:
      self.w_mfma.pop(r, None)
      self.w_trans.pop(r, None)
      (self.w_trans if trans else self.w_valu)[r] = self.now
    self._raw(text)

  def mfma(self, text, ab_reads=(), writes=()):
    need = 0
    for r in ab_reads:
      assert r in self.w_valu or r in self.w_trans, f"operand {r} not written yet"
      if r in self.w_valu: need = max(need, self.w_valu[r] + self.VALU_TO_MFMA)
      if r in self.w_trans: need = max(need, self.w_trans[r] + self.VALU_TO_MFMA)
      assert r not in self.w_mfma, f"matrix result {r} as A/B operand"
    self._pad_to(need)
    for r in writes:
      self.w_valu.pop(r, None)
      self.w_trans.pop(r, None)
      self.w_mfma[r] = self.now
    self._raw(text)

  def lds(self, text, tag, writes=()):
    self.lds_issued += 1
    self.tag_index[tag] = self.lds_issued
    for r in writes:
      self.w_valu.pop(r, None)
      self.w_trans.pop(r, None)
      assert r not in self.w_mfma or self.now - self.w_mfma[r] >= self.MFMA_TO_VALU, f"LDS read over a matrix result {r}"
      self.w_mfma.pop(r, None)
    self._raw(text)

  def need(self, *tags):
    want = max(self.tag_index[t] for t in tags)
    if want <= self.lds_done: return
    after = min(self.lds_issued - want, 15)
    self._raw(f"s_waitcnt lgkmcnt({after})")
    self.lds_done = self.lds_issued - after

  def text(self):
    return "".join(f'      "{l}\\n\\t"\n' for l in self.lines)


def vr(first, n=1):
  return f"v{first}" if n == 1 else f"v[{first}:{first + n - 1}]"


class PairGen:
  def __init__(self, base: int = 136, ablate=()):
    self.ablate = set(ablate)      # measurements only: "novalu", "nolds" leave instructions out (wrong results)
    b = base
    self.base = base
    self.ring = b; b += 4 * NRING
    self.s = [b, b + 32]; self.dp = [b + 16, b + 48]; b += 64       # S and dP of block 0 / 1 (u overwrites S)
    # P and dS of a block (bf16 pairs) take the place of its dP, half by half: rows 8 cc .. 8 cc + 7 of dP are read for
    # the last time just before P (registers 8 cc .. + 3) and dS (8 cc + 4 .. + 7) of those rows are formed
    self.pds = self.dp
    self.E = b; self.F = b + 8; self.G = b + 16; b += 24
    self.ra = b; b += 8                                              # row-read addresses; once the pair's last row read is out,
    self.ta = self.ra                                                # the transposing-read addresses [x][dvb] take their place
    self.end = b
    assert self.end <= 256, self.end
    self.em = Emitter()

  def clobbers(self):
    return [f"v{i}" for i in range(self.base, self.end)]

  # ---- addresses
  def row_addresses(self, blk):
    """ra[ks] = stage base + (a0 ^ 32 ks): the lane's 16 bytes of chunk 2 ks + half of its row, swizzled."""
    em = self.em
    for ks in range(8):
      r = self.ra + ks
      if ks == 0:
        em.valu(f"v_add_u32 {vr(r)}, %[sb], %[a0]", writes=(r,))
      else:
        em.valu(f"v_xor_b32 {vr(r)}, {32 * ks}, %[a0]", writes=(r,))
        em.valu(f"v_add_u32 {vr(r)}, %[sb], {vr(r)}", reads=(r,), writes=(r,))

  def tr_addresses(self):
    em = self.em
    for x in range(2):
      for dvb in range(4):
        r = self.ta + 4 * x + dvb
        k = (32 * x) ^ (64 * dvb)
        if k == 0:
          em.valu(f"v_add_u32 {vr(r)}, %[sb], %[t0]", writes=(r,))
        else:
          em.valu(f"v_xor_b32 {vr(r)}, {k}, %[t0]", writes=(r,))
          em.valu(f"v_add_u32 {vr(r)}, %[sb], {vr(r)}", reads=(r,), writes=(r,))

  # ---- the 64 matrix instructions of the pair and the LDS reads that feed them
  def slot_info(self, i):
    """(kind, block, index within its group)"""
    if i < 32: return ("s" if (i % 16) < 8 else "dp", i // 16, i % 8)
    j = i - 32
    blk, j = j // 16, j % 16
    return ("dvk", blk, j)           # j = 8 cc + 2 dvb + (0: dV, 1: dK)

  def frag_read(self, i):
    em = self.em
    if "nolds" in self.ablate: return
    kind, blk, j = self.slot_info(i)
    dst = self.ring + 4 * (i % NRING)
    regs = tuple(range(dst, dst + 4))
    boff = blk * STAGE
    if kind in ("s", "dp"):
      off = boff + (Q_BYTES if kind == "dp" else 0)
      em.lds(f"ds_read_b128 {vr(dst, 4)}, {vr(self.ra + j)} offset:{off}", f"f{i}", writes=regs)
    else:
      cc, dvb, which = j // 8, (j % 8) // 2, j % 2
      tile = 0 if which == 1 else Q_BYTES        # dK reads the Q tile, dV the dO tile
      for x in range(2):
        off = boff + tile + (16 * cc + 8 * x) * D * 2
        em.lds(f"ds_read_b64_tr_b16 {vr(dst + 2 * x, 2)}, {vr(self.ta + 4 * x + dvb)} offset:{off}", f"f{i}",
               writes=regs[2 * x: 2 * x + 2])

  def matrix(self, i):
    em = self.em
    kind, blk, j = self.slot_info(i)
    a = self.ring + 4 * (i % NRING)
    if "nomfma" in self.ablate or ("nosdp" in self.ablate and i < 32) or ("nodvk" in self.ablate and i >= 32): return
    if "nolds" not in self.ablate: em.need(f"f{i}")
    if kind == "s" or kind == "dp":
      acc = (self.s if kind == "s" else self.dp)[blk]
      b = f"%[{'k' if kind == 's' else 'v'}{j}]"
      c = "0" if j == 0 else vr(acc, 16)
      em.mfma(f"v_mfma_f32_32x32x16_bf16 {vr(acc, 16)}, {vr(a, 4)}, {b}, {c}", writes=tuple(range(acc, acc + 16)))
    else:
      cc, dvb, which = j // 8, (j % 8) // 2, j % 2
      pd = self.pds[blk] + 8 * cc + (0 if which == 0 else 4)
      acc = f"%[{'dv' if which == 0 else 'dk'}{dvb}]"
      em.mfma(f"v_mfma_f32_32x32x16_bf16 {acc}, {vr(a, 4)}, {vr(pd, 4)}, {acc}", ab_reads=() if "novalu" in self.ablate else tuple(range(pd, pd + 4)))

  # ---- the vector part of one block: (emit function) in issue order, rows 0..15 then 16..31
  def valu_ops(self, blk):
    em = self.em
    s, dp, pds = self.s[blk], self.dp[blk], self.pds[blk]
    E, F, G = self.E, self.F, self.G
    ops = []
    def op(text, reads=(), writes=(), trans=False, tags=()):
      def run():
        if tags: em.need(*tags)
        em.valu(text, reads=reads, writes=writes, trans=trans)
      ops.append(run)
    for cc in range(2):
      u0, d0 = s + 8 * cc, dp + 8 * cc
      for r in range(8):
        op(f"v_mul_f32 {vr(u0 + r)}, %[alpha], {vr(u0 + r)}", reads=(u0 + r,), writes=(u0 + r,))
      for r in range(8): op(f"v_exp_f32 {vr(E + r)}, -{vr(u0 + r)}", reads=(u0 + r,), writes=(E + r,), trans=True)
      for r in range(8): op(f"v_add_f32 {vr(E + r)}, 1.0, {vr(E + r)}", reads=(E + r,), writes=(E + r,))
      for r in range(8): op(f"v_rcp_f32 {vr(G + r)}, {vr(E + r)}", reads=(E + r,), writes=(G + r,), trans=True)
      for r in range(8): op(f"v_mul_f32 {vr(E + r)}, {LN2_BITS}, {vr(u0 + r)}", reads=(u0 + r,), writes=(E + r,))
      for r in range(8): op(f"v_sub_f32 {vr(F + r)}, 1.0, {vr(G + r)}", reads=(G + r,), writes=(F + r,))
      for r in range(8): op(f"v_fma_f32 {vr(F + r)}, {vr(E + r)}, {vr(F + r)}, 1.0", reads=(E + r, F + r), writes=(F + r,))
      for r in range(8): op(f"v_mul_f32 {vr(F + r)}, {vr(G + r)}, {vr(F + r)}", reads=(G + r, F + r), writes=(F + r,))
      for r in range(8): op(f"v_mul_f32 {vr(G + r)}, {vr(u0 + r)}, {vr(G + r)}", reads=(u0 + r, G + r), writes=(G + r,))
      for r in range(8): op(f"v_mul_f32 {vr(E + r)}, {vr(d0 + r)}, {vr(F + r)}", reads=(d0 + r, F + r), writes=(E + r,))
      for j in range(4):
        op(f"v_cvt_pk_bf16_f32 {vr(pds + 8 * cc + j)}, {vr(G + 2 * j)}, {vr(G + 2 * j + 1)}", reads=(G + 2 * j, G + 2 * j + 1), writes=(pds + 8 * cc + j,))
      for j in range(4):
        op(f"v_cvt_pk_bf16_f32 {vr(pds + 8 * cc + 4 + j)}, {vr(E + 2 * j)}, {vr(E + 2 * j + 1)}", reads=(E + 2 * j, E + 2 * j + 1), writes=(pds + 8 * cc + 4 + j,))
    return ops

  def build(self):
    em = self.em
    self.row_addresses(0)
    for i in range(LEAD): self.frag_read(i)
    va, vb = self.valu_ops(0), self.valu_ops(1)
    if "novalu" in self.ablate: va, vb = [], []
    # where each block's vector instructions go: block 0 behind slots 8..31 -- its products with dP(0), the
    # 81st instruction on, not before slot 16 --, block 1 behind slots 32..55, its first half done by slot 47
    plan = {}
    def spread(ops, first, last):
      n = max(len(ops), 1)
      for k, o in enumerate(ops):
        slot = first + (k * (last - first + 1)) // n
        plan.setdefault(slot, []).append(o)
    spread(va, 8, 31)
    spread(vb, 32, 55)
    for i in range(64):
      self.matrix(i)
      for o in plan.get(i, ()): o()
      if i + LEAD < 64:
        if i + LEAD == 32: self.tr_addresses()       # (the last row read went out a slot ago)
        self.frag_read(i + LEAD)
    em._raw("s_waitcnt lgkmcnt(0)")
    # the compiler does not know of the matrix instructions in here: what it puts behind the statement (a copy of
    # an accumulator, say) must find the last product's result in place
    em._raw("s_nop 15", 16)
    return self


def asm_statement(g: PairGen) -> str:
  # accumulators in vector registers: as C / D operands of these matrix instructions accumulation registers
  # measured 4.5 times slower (about 140 cycles an instruction against 32); K and V fragments, read as B operands
  # only, live there without loss
  outs = [f'[dv{i}] "+v"(dva[{i}])' for i in range(4)] + [f'[dk{i}] "+v"(dka[{i}])' for i in range(4)]
  kvc = "a"
  ins = [f'[k{i}] "{kvc}"(hs_k[{i}])' for i in range(8)] + [f'[v{i}] "{kvc}"(hs_v[{i}])' for i in range(8)]
  ins += ['[sb] "s"(hs_sb)', '[alpha] "s"(hs_alpha)', '[a0] "v"(hs_a0)', '[t0] "v"(hs_t0)']
  clob = ['"memory"'] + [f'"{c}"' for c in g.clobbers()]
  return (f"  asm volatile(\n{g.em.text()}"
          f"      : {', '.join(outs)}\n      : {', '.join(ins)}\n      : {', '.join(clob)});\n")


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "hstu_bwd_stream_d128.inc"))
  ap.add_argument("--base", type=int, default=136)
  ap.add_argument("--ablate", default="", help="measurements only, wrong results: comma-separated of novalu, nolds, nomfma, nosdp (no S / dP products), nodvk (no dV / dK products)")
  a = ap.parse_args()
  parts = ["// Generated by gen_bwd_stream.py: do not edit.  The hand-scheduled stream of the dK/dV kernel's interior blocks, a pair at a time.\n",
           "#define HSTU_BWD_STREAM_PAIR 1\n"]
  for name in ("HSTU_BWD_STREAM_PAIR",):
    g = PairGen(a.base, ablate=[x for x in a.ablate.split(",") if x]).build()
    parts.append(f"#if HSTU_BWD_STREAM_VARIANT == {name}\n{asm_statement(g)}#endif\n")
    print(name, len(g.em.lines), "lines,", g.em.pads, "wait states padded, registers", g.base, "..", g.end - 1)
  with open(a.out, "w") as f:
    f.write("".join(parts))
  print("wrote", a.out)


if __name__ == "__main__":
  main()
