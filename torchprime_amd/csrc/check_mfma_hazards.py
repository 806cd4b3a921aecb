#!/usr/bin/env python3
"""Build-time check of the gfx950 assembly that hipcc keeps beside an object file (-save-temps=obj).

A matrix instruction may read an A/B operand register that a vector-ALU instruction wrote only after two wait
states.  The compiler inserts them for the MFMAs it emits itself; it cannot look inside an ``asm`` statement, and it
is free to sink the instruction that packs an operand right in front of one.  The attention backward kernels issue
their accumulating MFMAs from ``asm`` statements (accumulators pinned to the accumulation registers), so every build
scans them: an MFMA inside an ASMSTART/ASMEND pair whose A or B registers were written by a vector-ALU instruction
fewer than two wait states earlier is reported and fails the build.

The other direction is checked too: the result registers of such an MFMA may be read by an ordinary instruction
only RESULT_WAIT_STATES later (a 32x32x16 MFMA writes them over its 16 passes).  The kernels read their pinned
accumulators only after the loop, behind explicit wait states; but where branches of a loop body end up with the
accumulators in different registers the compiler copies them (v_accvgpr_mov) right behind the MFMA, and such a copy
picks up registers that are not written yet.  Any read of an accumulation register within that distance of the asm
MFMA that writes it is reported.

Usage: check_mfma_hazards.py FILE.s [FILE.s ...]   (exit status 1 if anything is found)
"""
import re
import sys

REQUIRED_WAIT_STATES = 2
RESULT_WAIT_STATES = 19


def _vgprs(token):
  token = token.strip().rstrip(',')
  m = re.fullmatch(r'v\[(\d+):(\d+)\]', token)
  if m:
    return set(range(int(m.group(1)), int(m.group(2)) + 1))
  m = re.fullmatch(r'v(\d+)', token)
  return {int(m.group(1))} if m else set()


def _agprs(token):
  token = token.strip().rstrip(',')
  m = re.fullmatch(r'a\[(\d+):(\d+)\]', token)
  if m:
    return set(range(int(m.group(1)), int(m.group(2)) + 1))
  m = re.fullmatch(r'a(\d+)', token)
  return {int(m.group(1))} if m else set()


def _wait_states(instr):
  parts = instr.split()
  return int(parts[1], 0) + 1 if parts[0] == 's_nop' else 1


def _is_valu_write(op):
  return op.startswith('v_') and not op.startswith('v_mfma') and not op.startswith('v_accvgpr') and \
      not op.startswith('v_cmp') and not op.startswith('v_readfirstlane') and not op.startswith('v_readlane')


def scan(lines):
  """Returns [(kernel, line number, writer, mfma)] for every unprotected pair."""
  found, history, kernel, in_asm = [], [], None, False
  pending = []  # [agprs written by an asm MFMA, wait states since, its text]
  for number, raw in enumerate(lines, 1):
    text = raw.strip()
    if raw.startswith('_Z') and ':' in raw:
      kernel, history, pending = raw.split(':')[0], [], []
      continue
    if text.startswith(';;#ASMSTART'):
      in_asm = True
      continue
    if text.startswith(';;#ASMEND'):
      in_asm = False
      continue
    if not text or text.startswith(';') or text.startswith('.'):
      continue  # labels keep the history: the fall-through predecessor is the closest one
    text = text.split(';')[0].strip()
    op = text.split()[0]
    # reads of accumulation registers that an asm MFMA is still writing (an MFMA accumulating into the same
    # registers is the one reader the matrix unit interlocks itself)
    operands_all = [x.strip() for x in text[len(op):].split(',')] if len(text) > len(op) else []
    if not op.startswith('v_mfma'):
      reads = set()
      for tok in operands_all[1:]:
        reads |= _agprs(tok)
      for regs, waited, mfma in pending:
        if reads & regs and waited < RESULT_WAIT_STATES:
          found.append((kernel, number, mfma, text))
          break
    pending = [[regs, waited + _wait_states(text), mfma] for regs, waited, mfma in pending if waited + _wait_states(text) < RESULT_WAIT_STATES]
    if in_asm and op.startswith('v_mfma'):
      pending.append([_agprs(operands_all[0]), 0, text])
    if in_asm and op.startswith('v_mfma'):
      operands = [x.strip() for x in text[len(op):].split(',')]
      sources = _vgprs(operands[1]) | _vgprs(operands[2])
      waited = 0
      for prev in reversed(history):
        if waited >= REQUIRED_WAIT_STATES:
          break
        prev_op = prev.split()[0]
        if _is_valu_write(prev_op) and _vgprs(prev[len(prev_op):].split(',')[0]) & sources:
          found.append((kernel, number, prev, text))
          break
        waited += _wait_states(prev)
    history = (history + [text])[-8:]
  return found


def main(paths):
  total = 0
  for path in paths:
    with open(path) as f:
      found = scan(f)
    for kernel, number, writer, reader in found:
      n = RESULT_WAIT_STATES if writer.startswith('v_mfma') else REQUIRED_WAIT_STATES
      print(f'{path}:{number}: {kernel}: "{writer}" is less than {n} wait states ahead of "{reader}"')
    total += len(found)
  if total:
    print(f'{total} unprotected MFMA operand(s) / result(s): use the guarded form, move the writer away, or wait before the read')
  return 1 if total else 0


if __name__ == '__main__':
  sys.exit(main(sys.argv[1:]))
