#!/usr/bin/env python3
"""Build check for kernels whose matrix instructions are inline assembly.

The compiler does not know that such a statement is a matrix instruction and
counts no wait states behind it: a vector, LDS or memory instruction that
touches the instruction's result registers too soon reads (or is overwritten
by) a result that the matrix core has not written yet.  The kernels put their
own `s_nop` behind the last matrix instruction of a tile; this script reads the
compiler's assembly (`hipcc -S --cuda-device-only`) and fails if any other
instruction touches a matrix instruction's destination registers within
WINDOW instructions of it without such a wait in between -- which is what a
register copy that the compiler decided to insert there would look like.

usage: check_mfma_wait.py file.s
"""
import re
import sys

WINDOW = 20  # instructions; 16 passes need at most 18 wait states
REG = re.compile(r'\b([va])(?:(\d+)\b|\[([^\]]+)\])')


def _value(expr):
  if not re.fullmatch(r'[0-9a-fx+* ]+', expr):
    raise ValueError(expr)
  return int(eval(expr))  # digits, +, * only (checked above)


def registers(text):
  """{('v', 3), ...} named in an operand string."""
  out = set()
  for kind, single, inner in REG.findall(text):
    if single:
      out.add((kind, int(single)))
    elif ':' in inner:
      lo, hi = inner.split(':')
      out.update((kind, r) for r in range(_value(lo), _value(hi) + 1))
    else:
      out.add((kind, _value(inner)))
  return out


def main(path):
  pending = []  # [destination registers, instructions left]
  bad = 0
  for number, line in enumerate(open(path), 1):
    text = line.split(';')[0].strip()
    if not text or text.startswith('.') or text.endswith(':'):
      continue
    op, _, operands = text.partition(' ')
    if op.startswith('s_nop'):
      if _value(operands.strip()) >= 7:
        pending = []
      else:
        pending = [[d, n - 1] for d, n in pending if n > 1]
      continue
    if op.startswith('v_mfma'):
      # a matrix instruction may follow one on the same accumulator at once
      dst = registers(operands.split(',')[0])
      pending = [[d, n - 1] for d, n in pending if n > 1 and not (d & dst)]
      pending.append([dst, WINDOW])
      continue
    touched = registers(operands)
    for d, _ in pending:
      if d & touched:
        print(f'{path}:{number}: `{text}` touches the result of a matrix '
              f'instruction issued fewer than {WINDOW} instructions before it')
        bad += 1
        break
    pending = [[d, n - 1] for d, n in pending if n > 1]
  return 1 if bad else 0


if __name__ == '__main__':
  sys.exit(main(sys.argv[1]))
