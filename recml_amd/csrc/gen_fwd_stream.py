#!/usr/bin/env python3
"""Writes the hand-scheduled instruction stream of the forward kernel's interior blocks.

The forward kernel (hstu_attn.hip, hstu_fwd_mfma_bf16 at d = 128, bf16) spends its time in
32 x 32 blocks: 8 matrix instructions for the logits S^T = K Q^T, the pointwise part
(scale + bias, exp2, add, rcp, mul, pack: 88 vector instructions per lane-block of 16 logits),
8 matrix instructions for O^T += V^T P^T, 24 to 28 LDS fragment reads.  Written as C++ the
compiler orders them as three phases per block.  This generator emits the steady state as ONE
instruction stream per wave in which every matrix instruction is followed by its share of the
vector and LDS instructions of OTHER blocks (a software pipeline two blocks deep), with
registers assigned by hand, waits counted by hand and the wait states the hardware does not
interlock inserted by hand.

One iteration i of the stream (16 slots, one matrix instruction each):

  slots  0.. 3   O^T += V(i-1)[keys 16..31]^T P(i-1)[keys 16..31]      (fragments read in iteration i-1)
  slots  4..11   S(i+1)^T = K(i+1) Q^T
  slots 12..15   O^T += V(i)[keys 0..15]^T P(i)[keys 0..15]
  vector:        u(i) = alpha' S(i) + bias(i) first, then the SiLU of keys 0..15 -> P(i) low half
                 (needed by slot 12) and of keys 16..31 -> P(i) high half (needed by the next slot 0)
  LDS reads:     K(i+1), V(i), the position window of step i+1, each a few slots ahead of its use

so iteration i touches ring stage i % 4 for V and stage (i + 1) % 4 for K and the bias operands:
the K side of the ring runs one step ahead of the V side.  Iterations come in pairs with one
workgroup barrier per pair; the direct global->LDS loads of a pair go out right behind the
barrier: K (and bias operands) of steps 2j+3, 2j+4 and V of steps 2j+2, 2j+3 at the start of
pair j = iterations (2j, 2j+1).

Wait states written out by hand (gfx950; the assembler does not add them inside inline assembly):
  matrix instruction (8 passes) -> vector read of its result      11
  vector write -> matrix instruction read                          2
  exp2 / rcp result -> other vector instruction                    1
  write of m0 -> direct load                                       1

A wave without query rows (all 32 past the sequence's end) takes loads_only_variant instead: the loads,
waits and barriers of full_variant in the same order and number, and none of its arithmetic.

Usage:  python gen_fwd_stream.py [--out hstu_fwd_stream_d128.inc] [--experiments FILE]
The output is C++ source: `asm volatile(...)` statements for the kernel to #include, one per
variant (HSTU_STREAM_VARIANT selects which the including code expands).
"""

from __future__ import annotations

import argparse
import os

D = 128
STAGE = 16384          # bytes of one ring stage: K tile (8 KB) then V tile (8 KB)
K_BYTES = 8192
NSTAGE = 4
POS_BYTES = 2624       # 4 shifted copies of the position window (MfmaSmem::POS_BYTES)


class Regs:
  """The stream's own registers from v[base] up.  With `alias` the K fragments share registers with
  the V fragments of keys 0..15 and with the position window (96 registers), else 128."""

  def __init__(self, base: int, alias: bool, lag: bool = False, ts: bool = False):
    assert base % 4 == 0
    self.base = base
    b = base
    self.sacc = b; b += 16        # S^T accumulator of the block ahead
    self.u = b; b += 16           # scaled + biased logits of the block at hand
    if lag:
      # the schedule with P V one whole block behind: one set of 8 fragments that K and V take in turn,
      # P of two blocks, a temporary per logit
      self.e = b; b += 16
      self.p = [b, b + 8]; b += 16   # P of even / odd iterations, keys 0..15 then 16..31
      self.frag = b; b += 32
      self.posw = b; b += 16
      self.kf = self.frag
      self.dummy = b; b += 4        # (ablations only)
      self.end = b
      assert self.end <= 256
      return
    self.e = b; b += 8            # the SiLU's temporaries
    self.p0 = b; b += 4           # P, keys 0..15 (B operand)
    self.p1 = b; b += 4           # P, keys 16..31
    self.kf = b; b += 32          # K fragments 0..7
    self.vfb = b; b += 16         # V fragments of keys 16..31
    if alias:
      self.vfa = self.kf          # V fragments of keys 0..15: the registers of K fragments 0..3
      self.posw = self.kf + 16    # position window: those of K fragments 4..7
    else:
      self.vfa = b; b += 16
      self.posw = b; b += 16
    # timestamp bias: the lane's descriptor, its count of far keys (less 4 * half), the two table values, two scratch
    if ts:
      self.dsc = b; self.cp = b + 1; self.vn = b + 2; self.vf = b + 3; self.sel = b + 4; b += 6
    self.end = b
    assert self.end <= 256

  def r(self, first: int, n: int = 1) -> str:
    return f"v{first}" if n == 1 else f"v[{first}:{first + n - 1}]"

  def clobbers(self):
    return [f"v{i}" for i in range(self.base, self.end)]


class Stream:
  """Collects instructions, counts LDS reads in flight and puts the waits in."""

  def __init__(self, ablate=()):
    self.lines = []
    self.lds_issued = 0            # LDS instructions issued so far
    self.lds_done = 0              # ... of which known complete (waited for)
    self.tag_index = {}            # tag -> index (1-based) of the LDS read that defines it
    self.ablate = set(ablate)

  def emit(self, s: str):
    self.lines.append(s)

  def lds(self, s: str, tag: str):
    if "nolds" in self.ablate: return
    self.lds_issued += 1
    self.tag_index[tag] = self.lds_issued
    self.emit(s)

  def need(self, *tags: str):
    """Waits until the LDS reads behind the tags have landed (they complete in order)."""
    if "nolds" in self.ablate: return
    want = max(self.tag_index[t] for t in tags)
    if want <= self.lds_done:
      return
    after = min(self.lds_issued - want, 15)     # the counter's range: beyond it the wait is stricter than needed
    if "nowait" not in self.ablate: self.emit(f"s_waitcnt lgkmcnt({after})")
    self.lds_done = self.lds_issued - after

  def wait_all_lds(self):
    if self.lds_done < self.lds_issued:
      self.emit("s_waitcnt lgkmcnt(0)")
      self.lds_done = self.lds_issued

  def text(self) -> str:
    return "".join(f'      "{l}\\n\\t"\n' for l in self.lines)


def mfma(dst: str, a: str, b: str, c: str) -> str:
  return f"v_mfma_f32_32x32x16_bf16 {dst}, {a}, {b}, {c}"


# Where the LDS reads of an iteration are issued: slot -> list of groups, each placed behind the slot's
# matrix instruction and vector instructions (slot -1: ahead of slot 0).  "k0": K fragments 0..3 of the
# block ahead, "k1": 4..7, "va0" / "va1": V fragments of keys 0..15 (O blocks 0, 1 / 2, 3), "vb0" / "vb1":
# keys 16..31, "pos": the window.
# With shared registers the order is forced: k0 after the last product that reads the V fragments of keys
# 0..15 (slot 15 of the iteration before), k1 after the scale + bias instructions have read the window,
# va* after the logits' instructions that read K fragments 0..3, pos after those of 4..7.
LDS_SLOTS_ALIAS = {-1: ["k0"], 2: ["k1"], 8: ["va0"], 9: ["va1"], 10: ["vb0"], 11: ["vb1"], 13: ["pos"]}
# Without sharing everything goes out as early as its ring stage and its registers allow: K fragments of
# the block ahead right away (their last readers were slots 4..11 of the iteration before), V fragments of
# keys 0..15 (last read in slots 12..15 of the iteration before) behind them, keys 16..31 (read in slots
# 0..3) from slot 4, the window (read by the first vector instructions) last.
LDS_SLOTS_DEEP = {-1: ["k0", "k1"], 1: ["va0"], 2: ["va1"], 5: ["vb0"], 6: ["vb1"], 9: ["pos"]}


class Gen:
  def __init__(self, pos: bool, dma: bool, base: int = 160, alias: bool = True, lds_slots=None, valu: str = "phases", ablate=(),
               lag: bool = False, pos_slot: int = 11, ts: bool = False):
    self.pos = pos
    self.ts = ts
    self.dma = dma
    self.lag = lag
    self.pos_slot = pos_slot
    self.parity = 0               # lag schedule: which P buffer the iteration at hand writes
    self.R = Regs(140 if lag else base, alias, lag, ts)
    self.S = Stream(ablate)
    self.alias = alias
    self.lds_slots = lds_slots or (LDS_SLOTS_ALIAS if alias else LDS_SLOTS_DEEP)
    self.valu = valu
    self.ablate = set(ablate)

  # ---- operands by name (the including code binds them)
  def o(self, d): return f"%[o{d}]"
  def q(self, ks): return f"%[q{ks}]"
  def ka(self, ks): return f"%[ka{ks}]"
  def va(self, d): return f"%[va{d}]"

  @property
  def bias_stage(self):
    """Bytes of one ring stage's bias operands (the kernel's BIAS_STAGE).  With timestamps: four times (window
    copy | 64 bytes of descriptors), then 144 bytes of key timestamps."""
    if self.ts: return 4 * ((656 if self.pos else 0) + 64) + 144
    return POS_BYTES if self.pos else 0

  # ---- timestamp bias from descriptors
  def desc_read(self, kst: int):
    R, S = self.R, self.S
    S.lds(f"ds_read_u16 {R.r(R.dsc)}, %[dsa] offset:{kst * self.bias_stage}", "dsc")

  def desc_unpack(self):
    """bucket -> address of its table value; count of far keys less 4 * half."""
    R, S = self.R, self.S
    S.need("dsc")
    S.emit(f"v_and_b32 {R.r(R.sel)}, 127, {R.r(R.dsc)}")
    S.emit(f"v_bfe_u32 {R.r(R.cp)}, {R.r(R.dsc)}, 7, 6")
    S.emit(f"v_lshl_add_u32 {R.r(R.sel)}, {R.r(R.sel)}, 2, %[tva]")
    S.emit(f"v_sub_u32 {R.r(R.cp)}, {R.r(R.cp)}, %[hh4]")

  def value_read(self):
    R, S = self.R, self.S
    S.lds(f"ds_read2_b32 {R.r(R.vn, 2)}, {R.r(R.sel)} offset1:1", "tsv")

  def ts_ops(self, r: int):
    """u[r] += the far value when the key's index in the step, 4 half + 8 (r / 4) + r % 4, is below the count."""
    R = self.R
    sel = R.sel + (r & 1)
    return [(f"v_cmp_lt_i32 vcc, {8 * (r >> 2) + (r & 3)}, {R.r(R.cp)}", ("tsv",)),
            (f"v_cndmask_b32 {R.r(sel)}, {R.r(R.vn)}, {R.r(R.vf)}, vcc", ()),
            (f"v_add_f32 {R.r(R.u + r)}, {R.r(R.u + r)}, {R.r(sel)}", ())]

  # ---- the pieces of an iteration
  def k_reads(self, kst: int, lo: int, hi: int):
    R, S = self.R, self.S
    for ks in range(lo, hi):
      if "nok" in self.ablate:
        S.tag_index[f"k{ks}"] = S.lds_done
        continue
      dst = R.dummy if "ldsdummy" in self.ablate else R.kf + 4 * ks
      S.lds(f"ds_read_b128 {R.r(dst, 4)}, {self.ka(ks)} offset:{kst * STAGE}", f"k{ks}")

  def v_reads(self, vst: int, cc: int, dvbs):
    R, S = self.R, self.S
    dst0 = R.vfa if cc == 0 else R.vfb
    for d in dvbs:
      for x in range(2):
        off = vst * STAGE + (16 * cc + 8 * x) * D * 2
        S.lds(f"ds_read_b64_tr_b16 {R.r(dst0 + 4 * d + 2 * x, 2)}, {self.va(d)} offset:{off}", f"v{cc}{d}{x}")

  def pos_reads(self, kst: int):
    R, S = self.R, self.S
    for g in range(4):
      S.lds(f"ds_read_b128 {R.r(R.posw + 4 * g, 4)}, %[pa] offset:{kst * self.bias_stage + 32 * g}", f"p{g}")

  def lds_group(self, name: str, vst: int, kst: int, last: bool):
    if name == "k0":
      if not last: self.k_reads(kst, 0, 4)
    elif name == "k1":
      if not last: self.k_reads(kst, 4, 8)
    elif name == "va0": self.v_reads(vst, 0, (0, 1))
    elif name == "va1": self.v_reads(vst, 0, (2, 3))
    elif name == "vb0": self.v_reads(vst, 1, (0, 1))
    elif name == "vb1": self.v_reads(vst, 1, (2, 3))
    elif name == "pos":
      if self.pos and not last: self.pos_reads(kst)
    else:
      raise ValueError(name)

  def valu_ops(self):
    """The 88 vector instructions of one block in issue order, as (text, LDS tags needed)."""
    R = self.R
    U, E, A, RC, M, P = [], [], [], [], [], []
    for r in range(16):
      if self.pos:
        U.append((f"v_fma_f32 {R.r(R.u + r)}, {R.r(R.sacc + r)}, %[alpha], {R.r(R.posw + r)}", (f"p{r // 4}",)))
      else:
        U.append((f"v_mul_f32 {R.r(R.u + r)}, %[alpha], {R.r(R.sacc + r)}", ()))
    # the temporaries: 8 registers, element r of half cc uses e[r]
    for cc in range(2):
      u0 = R.u + 8 * cc
      E.append([(f"v_exp_f32 {R.r(R.e + r)}, -{R.r(u0 + r)}", ()) for r in range(8)])
      A.append([(f"v_add_f32 {R.r(R.e + r)}, 1.0, {R.r(R.e + r)}", ()) for r in range(8)])
      RC.append([(f"v_rcp_f32 {R.r(R.e + r)}, {R.r(R.e + r)}", ()) for r in range(8)])
      M.append([(f"v_mul_f32 {R.r(R.e + r)}, {R.r(u0 + r)}, {R.r(R.e + r)}", ()) for r in range(8)])
      p = R.p0 if cc == 0 else R.p1
      P.append([(f"v_cvt_pk_bf16_f32 {R.r(p + j)}, {R.r(R.e + 2 * j)}, {R.r(R.e + 2 * j + 1)}", ()) for j in range(4)])
    if self.valu == "phases":
      # scale + bias of all 16, then per half: (the timestamp bias of its 8,) 8 exp2, 8 add, 8 rcp, 8 mul, 4 pack
      ops = list(U)
      for cc in range(2):
        if self.ts:
          for r in range(8 * cc, 8 * cc + 8): ops += self.ts_ops(r)
        ops += E[cc] + A[cc] + RC[cc] + M[cc] + P[cc]
      return ops
    raise ValueError(self.valu)

  def iteration(self, vst: int, *, first_of_pair: bool, dma_lines=(), last: bool = False):
    """Iteration with V stage vst (K side: vst + 1).  `last`: no block ahead (no logits, no K / window reads)."""
    R, S = self.R, self.S
    kst = (vst + 1) % NSTAGE
    ops = self.valu_ops() if "novalu" not in self.ablate else []
    n_ops = len(ops)
    # vector instructions per slot, as even as 88 (136 with timestamps) over 16 goes
    per_slot = [(n_ops * (s + 1)) // 16 - (n_ops * s) // 16 for s in range(16)]
    pos_in_ops = 0
    if first_of_pair:
      for l in dma_lines: S.emit(l)
    for g in self.lds_slots.get(-1, ()): self.lds_group(g, vst, kst, last)
    for slot in range(16):
      # ---- the matrix instruction
      if slot < 4:
        d = slot
        if f"v1{d}1" in S.tag_index: S.need(f"v1{d}0", f"v1{d}1")
        S.emit(mfma(self.o(d), R.r(R.vfb + 4 * d, 4), R.r(R.p1, 4), self.o(d)))
      elif slot < 12:
        ks = slot - 4
        if not last:
          S.need(f"k{ks}")
          S.emit(mfma(R.r(R.sacc, 16), R.r(R.kf + 4 * ks, 4), self.q(ks), "0" if ks == 0 else R.r(R.sacc, 16)))
      else:
        d = slot - 12
        S.need(f"v0{d}0", f"v0{d}1")
        S.emit(mfma(self.o(d), R.r(R.vfa + 4 * d, 4), R.r(R.p0, 4), self.o(d)))
      # ---- this slot's vector instructions
      for _ in range(per_slot[slot]):
        ins, tags = ops[pos_in_ops]
        pos_in_ops += 1
        if tags: S.need(*tags)
        S.emit(ins)
      # ---- LDS reads placed behind the vector instructions of a slot
      for g in self.lds_slots.get(slot, ()):
        if g == "k1" and self.alias and n_ops: assert pos_in_ops >= 16   # the window's registers are free
        self.lds_group(g, vst, kst, last)
      if self.ts and not last:
        # the next block's descriptor: read early, unpacked once this block's timestamp instructions are out
        # (they use the same registers), its two table values asked for right behind
        if slot == 3: self.desc_read(kst)
        if slot == 11:
          assert pos_in_ops >= 16 + 48 + 36
          self.desc_unpack()
          self.value_read()
    assert pos_in_ops == n_ops

  def valu_ops_lag(self, pcur: int):
    """The block's 88 vector instructions for the schedule with P V a block behind: scale + bias of all 16
    logits, then the four quads of logits through exp2, add, rcp, mul, pack one step behind each other, a
    quad's slow instructions (exp2, rcp) between its neighbours' fast ones.  Every logit has its own
    temporary; a dependent instruction is at least 4 instructions behind its producer."""
    R = self.R
    seq = []
    for r in range(16):
      if self.pos:
        seq.append((f"v_fma_f32 {R.r(R.u + r)}, {R.r(R.sacc + r)}, %[alpha], {R.r(R.posw + r)}", (f"p{r // 4}",)))
      else:
        seq.append((f"v_mul_f32 {R.r(R.u + r)}, %[alpha], {R.r(R.sacc + r)}", ()))
    def E(q): return [(f"v_exp_f32 {R.r(R.e + r)}, -{R.r(R.u + r)}", ()) for r in range(4 * q, 4 * q + 4)]
    def A(q): return [(f"v_add_f32 {R.r(R.e + r)}, 1.0, {R.r(R.e + r)}", ()) for r in range(4 * q, 4 * q + 4)]
    def RC(q): return [(f"v_rcp_f32 {R.r(R.e + r)}, {R.r(R.e + r)}", ()) for r in range(4 * q, 4 * q + 4)]
    def M(q): return [(f"v_mul_f32 {R.r(R.e + r)}, {R.r(R.u + r)}, {R.r(R.e + r)}", ()) for r in range(4 * q, 4 * q + 4)]
    def P(q): return [(f"v_cvt_pk_bf16_f32 {R.r(pcur + 2 * q + j)}, {R.r(R.e + 4 * q + 2 * j)}, {R.r(R.e + 4 * q + 2 * j + 1)}", ()) for j in range(2)]
    for k in range(4 + 4):
      fast, slow = [], []
      for q in range(4):
        st = k - q
        if st == 0: slow += E(q)
        if st == 1: fast += A(q)
        if st == 2: slow += RC(q)
        if st == 3: fast += M(q)
        if st == 4: fast += P(q)
      n = max(len(slow), len(fast))
      for i in range(n):
        if i < len(slow): seq.append(slow[i])
        if i < len(fast): seq.append(fast[i])
    assert len(seq) == 88, len(seq)
    return seq

  def iteration_lag(self, vst: int, *, first_of_pair: bool, dma_lines=(), last: bool = False):
    """The schedule with P V one whole block behind.  Slots 0..7: O^T += V(i-1)^T P(i-1), fragments read in
    iteration i-1; behind slot f the K fragment f of block i+1 is read into the registers its V fragment has
    left.  Slots 8..15: S(i+1)^T = K(i+1) Q^T; behind slot 8+f the V fragment f of block i follows into the
    same registers.  Every fragment is asked for 8 slots ahead of its use.  The vector part is the whole
    SiLU of block i, due only at the iteration's end (P is double-buffered)."""
    R, S = self.R, self.S
    kst = (vst + 1) % NSTAGE
    pcur, pprev = R.p[self.parity], R.p[self.parity ^ 1]
    self.parity ^= 1
    ops = self.valu_ops_lag(pcur) if "novalu" not in self.ablate else []
    n_ops = len(ops)
    per_slot = [(n_ops * (s + 1)) // 16 - (n_ops * s) // 16 for s in range(16)]
    pos_in_ops = 0
    if first_of_pair:
      for l in dma_lines: S.emit(l)
    for slot in range(16):
      if slot < 8:
        f = slot
        cc, d = f // 4, f % 4
        if f"vf{f}1" in S.tag_index: S.need(f"vf{f}0", f"vf{f}1")
        S.emit(mfma(self.o(d), R.r(R.frag + 4 * f, 4), R.r(pprev + 4 * cc, 4), self.o(d)))
      else:
        ks = slot - 8
        if not last:
          S.need(f"k{ks}")
          S.emit(mfma(R.r(R.sacc, 16), R.r(R.frag + 4 * ks, 4), self.q(ks), "0" if ks == 0 else R.r(R.sacc, 16)))
      for _ in range(per_slot[slot]):
        ins, tags = ops[pos_in_ops]
        pos_in_ops += 1
        if tags: S.need(*tags)
        S.emit(ins)
      if slot < 8:
        if not last: self.k_reads(kst, slot, slot + 1)
      else:
        f = slot - 8
        cc, d = f // 4, f % 4
        for x in range(2):
          off = vst * STAGE + (16 * cc + 8 * x) * D * 2
          if "nov" in self.ablate or ("vb128" in self.ablate and x == 1):
            S.tag_index[f"vf{f}{x}"] = S.lds_done
            continue
          dst = R.dummy + 2 * x if "ldsdummy" in self.ablate else R.frag + 4 * f + 2 * x
          if "vb128" in self.ablate:
            S.lds(f"ds_read_b128 {R.r(R.frag + 4 * f, 4)}, {self.ka(f)} offset:{vst * STAGE + K_BYTES}", f"vf{f}{x}")
          else:
            S.lds(f"ds_read_b64_tr_b16 {R.r(dst, 2)}, {self.va(d)} offset:{off}", f"vf{f}{x}")
      if slot == self.pos_slot and self.pos and not last:
        assert pos_in_ops >= 16
        self.pos_reads(kst)
    assert pos_in_ops == n_ops

  def prologue_lag(self, kst: int):
    R, S = self.R, self.S
    for r in range(16): S.emit(f"v_mov_b32 {R.r(R.p[0] + r)}, 0")
    self.k_reads(kst, 0, 8)
    for ks in range(8):
      S.need(f"k{ks}")
      S.emit(mfma(R.r(R.sacc, 16), R.r(R.frag + 4 * ks, 4), self.q(ks), "0" if ks == 0 else R.r(R.sacc, 16)))
    if self.pos: self.pos_reads(kst)
    # the first iteration's product has an all-zero P; its A operand must still be finite: zeros
    S.emit("s_nop 7")
    S.emit("s_nop 3")
    for r in range(32): S.emit(f"v_mov_b32 {R.r(R.frag + r)}, 0")
    self.parity = 0

  def tail_lag(self):
    R, S = self.R, self.S
    pprev = R.p[self.parity ^ 1]
    S.emit("s_nop 1")
    for f in range(8):
      cc, d = f // 4, f % 4
      if f"vf{f}1" in S.tag_index: S.need(f"vf{f}0", f"vf{f}1")
      S.emit(mfma(self.o(d), R.r(R.frag + 4 * f, 4), R.r(pprev + 4 * cc, 4), self.o(d)))
    S.wait_all_lds()
    S.emit("s_nop 7")
    S.emit("s_nop 7")
    S.emit("s_nop 3")

  def _load(self, L, dst_sgpr, imm, off, ptr):
    L.append(f"s_add_u32 m0, {dst_sgpr}, {imm}")
    L.append("s_nop 0")
    L.append(f"global_load_lds_dwordx4 {off}, {ptr}")

  def dma_k_side(self, st: int):
    """Direct loads of one step's K tile (and position window) into ring stage st; the scalar pointers
    s[90:91] (K rows) and s[94:95] (window) then move on by one step."""
    L = []
    for r in range(2): self._load(L, "%[kdst]", st * STAGE + r * 1024, f"%[koff{r}]", "s[90:91]")
    L.append("s_add_u32 s90, s90, %[kstep]")
    L.append("s_addc_u32 s91, s91, 0")
    if self.ts:
      # window, descriptors and key timestamps move on by different strides: a per-lane increment
      L.append("s_mov_b64 exec, %[bexec]")
      self._load(L, "%[bdst]", st * self.bias_stage, "%[boff]", "s[94:95]")
      L.append("v_add_u32 %[boff], %[boff], %[binc]")
      L.append("s_mov_b64 exec, -1")
    elif self.pos:
      L.append("s_mov_b64 exec, %[bexec]")
      self._load(L, "%[bdst]", st * self.bias_stage, "%[boff]", "s[94:95]")
      L.append("s_mov_b64 exec, -1")
      L.append("s_add_u32 s94, s94, 128")
      L.append("s_addc_u32 s95, s95, 0")
    return L

  def dma_pair(self, vst: int):
    """Direct loads at the start of the pair whose first iteration has V stage vst (0 or 2): K and the bias
    operands of the steps three and four ahead, V of the steps two and three ahead.  s[90:91], s[92:93], s[94:95]
    are the scalar pointers (copies of %[kp], %[vp], %[bp]) that walk along the rows, one step of 32 keys at a time."""
    L = []
    for ahead in (3, 4): L += self.dma_k_side((vst + ahead) % NSTAGE)
    for ahead in (2, 3):
      st = (vst + ahead) % NSTAGE
      for r in range(2): self._load(L, "%[vdst]", st * STAGE + r * 1024, f"%[voff{r}]", "s[92:93]")
      L.append("s_add_u32 s92, s92, %[vstep]")
      L.append("s_addc_u32 s93, s93, 0")
    return L

  def end_of_pair(self):
    """Every load of this wave has landed and every LDS read of it is done; then the workgroup meets."""
    S = self.S
    S.emit("s_waitcnt vmcnt(0) lgkmcnt(0)")
    S.lds_done = S.lds_issued
    S.emit("s_barrier")

  def prologue(self, kst: int):
    """Logits of the first block (K side stage kst) with nothing to overlap, empty pending product."""
    R, S = self.R, self.S
    for r in range(4): S.emit(f"v_mov_b32 {R.r(R.p1 + r)}, 0")
    for r in range(16): S.emit(f"v_mov_b32 {R.r(R.vfb + r)}, 0")
    self.k_reads(kst, 0, 8)
    for ks in range(8):
      S.need(f"k{ks}")
      S.emit(mfma(R.r(R.sacc, 16), R.r(R.kf + 4 * ks, 4), self.q(ks), "0" if ks == 0 else R.r(R.sacc, 16)))
    if self.pos: self.pos_reads(kst)
    if self.ts:
      self.desc_read(kst)
      self.desc_unpack()
      self.value_read()
    # the scale + bias instructions read the accumulator: 11 wait states behind the last matrix instruction
    S.emit("s_nop 7")
    S.emit("s_nop 3")

  def tail(self):
    """The product still pending after the last iteration, then wait states until the accumulators may be read."""
    R, S = self.R, self.S
    for d in range(4):
      if f"v1{d}1" in S.tag_index: S.need(f"v1{d}0", f"v1{d}1")
      if d == 0: S.emit("s_nop 1")     # vector write of P -> matrix read
      S.emit(mfma(self.o(d), R.r(R.vfb + 4 * d, 4), R.r(R.p1, 4), self.o(d)))
    S.wait_all_lds()
    S.emit("s_nop 7")
    S.emit("s_nop 7")
    S.emit("s_nop 3")


def compute_only_variant(pos: bool, base: int, **kw) -> Gen:
  """A loop of 4 iterations over the ring with no loads and no barrier (LDS filled beforehand): the
  measurement of the stream's own issue time.  %[n] counts rounds of 4 iterations."""
  g = Gen(pos, dma=False, base=base, **kw)
  S = g.S
  (g.prologue_lag if g.lag else g.prologue)(0)
  S.wait_all_lds()
  S.emit("1:")
  for it in range(4):
    (g.iteration_lag if g.lag else g.iteration)(it % NSTAGE, first_of_pair=(it % 2 == 0))
    S.emit("s_nop 1")    # the next iteration's first product reads P, written by this one's last vector instructions
  S.wait_all_lds()
  S.emit("s_sub_u32 %[n], %[n], 1")
  S.emit("s_cmp_lg_u32 %[n], 0")
  S.emit("s_cbranch_scc1 1b")
  (g.tail_lag if g.lag else g.tail)()
  return g


def full_variant(pos: bool, base: int, **kw) -> Gen:
  """The stream as the kernel runs it: %[n] >= 1 rounds of two pairs of iterations, loads behind each pair's
  barrier.  On entry the tiles (and bias operands) of steps 0 and 1 are in ring stages 0 and 1 and published,
  nothing else is in flight, every other stage is free: what the kernel's paired loop expects at the start of
  a pair, so the stream can take over at any pair that begins at stage 0.  Its first pair also sends for the K
  side of step 2, ahead of its own loads, and the workgroup meets once more between that pair's two iterations
  to publish it.  On exit the tiles of V steps 4n, 4n+1 and K steps 4n .. 4n+2 are in the ring and published."""
  g = Gen(pos, dma=True, base=base, **kw)
  S = g.S
  S.emit("s_mov_b64 s[90:91], %[kp]")
  S.emit("s_mov_b64 s[92:93], %[vp]")
  if pos or g.ts: S.emit("s_mov_b64 s[94:95], %[bp]")
  (g.prologue_lag if g.lag else g.prologue)(0)
  # The first pair's loads overwrite ring stage 0 on the K side (the tile and window of step 4), which every
  # wave has just read for the first block's logits: they wait for each other before any of them sends for it.
  S.wait_all_lds()
  S.emit("s_barrier")
  it = g.iteration_lag if g.lag else g.iteration
  def quad(first: bool):
    for pair in range(2):
      vst = 2 * pair
      lines = g.dma_pair(vst)
      if first and pair == 0:
        # K side of step 2 into stage 2 first ([kp], [bp] point at step 2 on entry), then the pair's own loads
        lines = g.dma_k_side(2) + lines
      it(vst, first_of_pair=True, dma_lines=lines)
      if first and pair == 0:
        # this wave's share of step 2's K side has landed once at most the pair's own loads are in flight
        own = (3 if (pos or g.ts) else 2) * 2 + 2 * 2
        S.emit(f"s_waitcnt vmcnt({own})")
        S.emit("s_barrier")
      else:
        S.emit("s_nop 1")
      it(vst + 1, first_of_pair=False)
      g.end_of_pair()
  quad(True)
  S.emit("s_sub_u32 %[n], %[n], 1")
  S.emit("s_cmp_eq_u32 %[n], 0")
  S.emit("s_cbranch_scc1 2f")
  S.emit("1:")
  quad(False)
  S.emit("s_sub_u32 %[n], %[n], 1")
  S.emit("s_cmp_lg_u32 %[n], 0")
  S.emit("s_cbranch_scc1 1b")
  S.emit("2:")
  (g.tail_lag if g.lag else g.tail)()
  return g


def loads_only_variant(pos: bool, ts: bool) -> Gen:
  """What a wave without query rows (all 32 past the sequence's end) runs in place of full_variant: its share of the
  direct loads, the waits for them and every barrier of the workgroup, in the same order and number, and nothing else.
  A pair's loads go to ring stages whose last readers finished before the barrier that starts the pair, so they may
  all go out right behind it."""
  g = Gen(pos, dma=True, base=152 if ts else 160, ts=ts, **PRODUCT)     # (the register window goes unused)
  g.loads_only = True
  S = g.S = Stream()
  S.emit("s_mov_b64 s[90:91], %[kp]")
  S.emit("s_mov_b64 s[92:93], %[vp]")
  if pos or ts: S.emit("s_mov_b64 s[94:95], %[bp]")
  S.emit("s_barrier")                      # (full_variant: behind the first block's logits)
  def quad(first: bool):
    for pair in range(2):
      vst = 2 * pair
      lines = g.dma_pair(vst)
      if first and pair == 0: lines = g.dma_k_side(2) + lines
      for l in lines: S.emit(l)
      if first and pair == 0:
        own = (3 if (pos or ts) else 2) * 2 + 2 * 2
        S.emit(f"s_waitcnt vmcnt({own})")
        S.emit("s_barrier")
      S.emit("s_waitcnt vmcnt(0)")
      S.emit("s_barrier")
  quad(True)
  S.emit("s_sub_u32 %[n], %[n], 1")
  S.emit("s_cmp_eq_u32 %[n], 0")
  S.emit("s_cbranch_scc1 2f")
  S.emit("1:")
  quad(False)
  S.emit("s_sub_u32 %[n], %[n], 1")
  S.emit("s_cmp_lg_u32 %[n], 0")
  S.emit("s_cbranch_scc1 1b")
  S.emit("2:")
  return g


def asm_statement(g: Gen) -> str:
  if getattr(g, "loads_only", False):
    ins = ['[kdst] "s"(hs_kdst)', '[vdst] "s"(hs_vdst)', '[kstep] "s"(hs_kstep)', '[vstep] "s"(hs_vstep)']
    ins += [f'[koff{r}] "v"(hs_koff[{r}])' for r in range(2)] + [f'[voff{r}] "v"(hs_voff[{r}])' for r in range(2)]
    ins += ['[kp] "s"(hs_kp)', '[vp] "s"(hs_vp)']
    outs = ['[n] "+s"(hs_n)']
    if g.ts:
      ins += ['[bdst] "s"(hs_bdst)', '[binc] "v"(hs_binc)', '[bexec] "s"(hs_bexec)', '[bp] "s"(hs_bp)']
      outs.append('[boff] "+v"(hs_boff)')
    elif g.pos:
      ins += ['[bdst] "s"(hs_bdst)', '[boff] "v"(hs_boff)', '[bexec] "s"(hs_bexec)', '[bp] "s"(hs_bp)']
    clob = ['"memory"', '"scc"', '"m0"'] + [f'"s{i}"' for i in range(90, 96)]
    return (f"  asm volatile(\n{g.S.text()}"
            f"      : {', '.join(outs)}\n      : {', '.join(ins)}\n      : {', '.join(clob)});\n")
  ins = ['[alpha] "s"(hs_alpha)']
  ins += [f'[q{ks}] "v"(hs_q[{ks}])' for ks in range(8)]
  ins += [f'[ka{ks}] "v"(hs_ka[{ks}])' for ks in range(8)]
  ins += [f'[va{d}] "v"(hs_va[{d}])' for d in range(4)]
  if g.pos: ins.append('[pa] "v"(hs_pa)')
  if g.ts:
    ins += ['[dsa] "v"(hs_dsa)', '[tva] "s"(hs_tva)', '[hh4] "v"(hs_hh4)']
    clob_extra = ['"vcc"']
  else:
    clob_extra = []
  outs = [f'[o{d}] "+v"(hs_o[{d}])' for d in range(4)] + ['[n] "+s"(hs_n)']
  clob = ['"memory"', '"scc"'] + clob_extra + [f'"{c}"' for c in g.R.clobbers()]
  if g.dma:
    ins += ['[kdst] "s"(hs_kdst)', '[vdst] "s"(hs_vdst)', '[kstep] "s"(hs_kstep)', '[vstep] "s"(hs_vstep)']
    ins += [f'[koff{r}] "v"(hs_koff[{r}])' for r in range(2)] + [f'[voff{r}] "v"(hs_voff[{r}])' for r in range(2)]
    ins += ['[kp] "s"(hs_kp)', '[vp] "s"(hs_vp)']
    clob += ['"m0"'] + [f'"s{i}"' for i in range(90, 96)]
    if g.ts:
      ins += ['[bdst] "s"(hs_bdst)', '[binc] "v"(hs_binc)', '[bexec] "s"(hs_bexec)', '[bp] "s"(hs_bp)']
      outs.append('[boff] "+v"(hs_boff)')
    elif g.pos:
      ins += ['[bdst] "s"(hs_bdst)', '[boff] "v"(hs_boff)', '[bexec] "s"(hs_bexec)', '[bp] "s"(hs_bp)']
  return (f"  asm volatile(\n{g.S.text()}"
          f"      : {', '.join(outs)}\n      : {', '.join(ins)}\n      : {', '.join(clob)});\n")


def statement(g: Gen, name: str) -> str:
  return f"#if HSTU_STREAM_VARIANT == {name}\n{asm_statement(g)}#endif\n"


# What the product build takes (measured against the alternatives by --experiments).
PRODUCT = dict(alias=True, valu="phases")


def experiments(base_alias: int, base_deep: int):
  """(name, pos, wrong, full, generator) for the microbenchmark's sweep; `wrong` marks ablations that leave
  instructions out and compute wrong results on purpose."""
  ex = []
  def add(name, pos=False, wrong=False, full=False, **kw):
    base = base_alias if kw.get("alias", True) else base_deep
    g = (full_variant if full else compute_only_variant)(pos, base, **kw)
    ex.append((name, pos, wrong, full, g))
  add("shared registers, phases")
  add("shared registers, phases, no waits for LDS", wrong=True, ablate=("nowait",))
  add("shared registers, phases, no LDS reads", wrong=True, ablate=("nolds",))
  add("shared registers, phases, no vector instructions", wrong=True, ablate=("novalu",))
  add("matrix instructions only", wrong=True, ablate=("novalu", "nolds"))
  add("own registers, early reads, phases", alias=False)
  add("P V a block behind", lag=True)
  add("P V a block behind, no waits for LDS", wrong=True, lag=True, ablate=("nowait",))
  add("P V a block behind, no LDS reads", wrong=True, lag=True, ablate=("nolds",))
  add("P V a block behind, no vector instructions", wrong=True, lag=True, ablate=("novalu",))
  add("P V a block behind, no K reads", wrong=True, lag=True, ablate=("nok",))
  add("P V a block behind, no V reads", wrong=True, lag=True, ablate=("nov",))
  add("P V a block behind, V by 8 b128 reads", wrong=True, lag=True, ablate=("vb128",))
  add("P V a block behind, reads into registers nothing uses", wrong=True, lag=True, ablate=("ldsdummy",))
  add("P V a block behind, no vector instructions, no K reads", wrong=True, lag=True, ablate=("novalu", "nok"))
  add("P V a block behind, no vector instructions, no V reads", wrong=True, lag=True, ablate=("novalu", "nov"))
  add("P V a block behind, matrix instructions only", wrong=True, lag=True, ablate=("novalu", "nolds"))
  add("P V a block behind, window", pos=True, lag=True)
  add("shared registers, phases, window", pos=True)
  add("with loads: shared registers, phases", full=True)
  add("with loads: P V a block behind", full=True, lag=True)
  add("with loads: shared registers, phases, window", pos=True, full=True)
  add("with loads: P V a block behind, window", pos=True, full=True, lag=True)
  return ex


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "hstu_fwd_stream_d128.inc"))
  ap.add_argument("--base", type=int, default=160)
  ap.add_argument("--experiments", default=None, help="also write the sweep's variants (for micro_fwd_stream.hip -DHSTU_STREAM_EXPERIMENTS) to this file")
  a = ap.parse_args()
  parts = ["// Generated by gen_fwd_stream.py: do not edit.  The hand-scheduled stream of the forward kernel's interior blocks.\n",
           "#define HSTU_STREAM_COMPUTE_ONLY 1\n#define HSTU_STREAM_COMPUTE_ONLY_POS 2\n#define HSTU_STREAM_FULL 3\n#define HSTU_STREAM_FULL_POS 4\n"
           "#define HSTU_STREAM_FULL_TS 5\n#define HSTU_STREAM_FULL_POS_TS 6\n"
           "#define HSTU_STREAM_LOADS_ONLY 7\n#define HSTU_STREAM_LOADS_ONLY_POS 8\n#define HSTU_STREAM_LOADS_ONLY_TS 9\n"
           "#define HSTU_STREAM_LOADS_ONLY_POS_TS 10\n"]
  parts.append(statement(compute_only_variant(False, a.base, **PRODUCT), "HSTU_STREAM_COMPUTE_ONLY"))
  parts.append(statement(compute_only_variant(True, a.base, **PRODUCT), "HSTU_STREAM_COMPUTE_ONLY_POS"))
  parts.append(statement(full_variant(False, a.base, **PRODUCT), "HSTU_STREAM_FULL"))
  parts.append(statement(full_variant(True, a.base, **PRODUCT), "HSTU_STREAM_FULL_POS"))
  parts.append(statement(full_variant(False, a.base - 8, ts=True, **PRODUCT), "HSTU_STREAM_FULL_TS"))
  parts.append(statement(full_variant(True, a.base - 8, ts=True, **PRODUCT), "HSTU_STREAM_FULL_POS_TS"))
  parts.append(statement(loads_only_variant(False, False), "HSTU_STREAM_LOADS_ONLY"))
  parts.append(statement(loads_only_variant(True, False), "HSTU_STREAM_LOADS_ONLY_POS"))
  parts.append(statement(loads_only_variant(False, True), "HSTU_STREAM_LOADS_ONLY_TS"))
  parts.append(statement(loads_only_variant(True, True), "HSTU_STREAM_LOADS_ONLY_POS_TS"))    # (another pitch of the bias stages)
  with open(a.out, "w") as f:
    f.write("".join(parts))
  print("wrote", a.out)
  if a.experiments:
    ex = experiments(160, 128)
    with open(a.experiments, "w") as f:
      f.write("// Generated by gen_fwd_stream.py --experiments: the sweep's variants.\n")
      f.write(f"#define HSTU_EXP_COUNT {len(ex)}\n")
      f.write("#ifndef HSTU_EXP_TABLE\n")
      for i, (name, pos, wrong, full, g) in enumerate(ex):
        f.write(f"template <> __device__ __forceinline__ void hs_exp<{i}>(HS_PARAMS) {{\n{asm_statement(g)}}}\n")
      f.write("#else\n")
      for i, (name, pos, wrong, full, g) in enumerate(ex):
        f.write(f'  HSTU_EXP_ENTRY({i}, "{name}", {"true" if pos else "false"}, {"true" if wrong else "false"}, {"true" if full else "false"})\n')
      f.write("#endif\n")
    print("wrote", a.experiments, len(ex), "variants")


if __name__ == "__main__":
  main()
