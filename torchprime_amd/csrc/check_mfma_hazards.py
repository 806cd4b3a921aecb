#!/usr/bin/env python3
"""Build-time check of the gfx950 assembly that hipcc keeps beside an object file (-save-temps=obj).

A matrix instruction may read an A/B operand register that a vector-ALU instruction wrote only after two wait
states.  The compiler inserts them for the MFMAs it emits itself; it cannot look inside an ``asm`` statement, and it
is free to sink the instruction that packs an operand right in front of one.  The attention backward kernels issue
their accumulating MFMAs from ``asm`` statements (accumulators pinned to the accumulation registers), so every build
scans them: an MFMA inside an ASMSTART/ASMEND pair whose A or B registers were written by a vector-ALU instruction
fewer than two wait states earlier is reported and fails the build.

Usage: check_mfma_hazards.py FILE.s [FILE.s ...]   (exit status 1 if anything is found)
"""
import re
import sys

REQUIRED_WAIT_STATES = 2


def _vgprs(token):
  token = token.strip().rstrip(',')
  m = re.fullmatch(r'v\[(\d+):(\d+)\]', token)
  if m:
    return set(range(int(m.group(1)), int(m.group(2)) + 1))
  m = re.fullmatch(r'v(\d+)', token)
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
  for number, raw in enumerate(lines, 1):
    text = raw.strip()
    if raw.startswith('_Z') and ':' in raw:
      kernel, history = raw.split(':')[0], []
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
    for kernel, number, writer, mfma in found:
      print(f'{path}:{number}: {kernel}: "{writer}" is less than {REQUIRED_WAIT_STATES} wait states ahead of "{mfma}"')
    total += len(found)
  if total:
    print(f'{total} unprotected MFMA operand(s): use the guarded form or move the writer away')
  return 1 if total else 0


if __name__ == '__main__':
  sys.exit(main(sys.argv[1:]))
