#!/usr/bin/env python3
"""Build-time check of the machine code of spmm_rows.hip (run by the Makefile on the device pass's output).

The rows-along-lanes kernel names its vector registers outright inside inline assembly (v44 and up: three sets of
dense rows, the diagonal-value buffers, the sums, the halo) and loads into them asynchronously, across statement
boundaries.  The compiler knows of them only through clobber lists, so two things are outside its guarantees and
are verified here on the disassembly instead, before the code can reach a GPU:

  1. Register ownership.  No compiler-generated instruction may touch v44 or above, except lane spills of scalar
     registers into v76/v77 (which the kernel leaves free).  A compiler temporary in a register that has a load in
     flight is overwritten when the load lands -- with a buffer descriptor under construction in it, the next
     load goes to a wild address.
  2. Wait states the compiler does not pad around inline assembly on gfx950:
       VALU writes a VGPR   -> v_readfirstlane / v_readlane of it : 1 wait state
       v_readfirstlane / v_readlane writes an SGPR -> a VMEM instruction reads it : 5 wait states

Usage: check_rows_isa.py <bundle.hipfb | code-object> [--llvm-bin DIR]
Exit status 0 when every kernel in the file passes, 1 otherwise (with the offending instructions listed).
"""
import argparse
import collections
import os
import re
import subprocess
import sys
import tempfile

FIRST_OWNED = 44                 # RW_OWN2 in spmm_rows.hip: the lowest register the assembly names
SPILL_LANES = (76, 77)           # left free between the own sets and the value buffers
# what the assembly itself issues on the owned registers
ASM_OPS = {'v_fmac_f32_e32', 'v_mov_b32_dpp', 'ds_read_b128', 'buffer_load_dwordx4', 'buffer_load_dword',
           'ds_write_b128'}
ACC_FIRST = 112                  # RW_ACC: zeroed with v_mov_b32 v, 0 by the assembly


def disassemble(path, llvm_bin):
    with open(path, 'rb') as f:
        magic = f.read(24)
    with tempfile.TemporaryDirectory() as tmp:
        co = path
        if magic.startswith(b'__CLANG_OFFLOAD_BUNDLE__'):
            co = os.path.join(tmp, 'dev.co')
            listing = subprocess.run([os.path.join(llvm_bin, 'clang-offload-bundler'), '--list', '--type=o',
                                      '--input=' + path], check=True, capture_output=True, text=True).stdout.split()
            targets = [t for t in listing if 'amdgcn' in t]
            if len(targets) != 1:
                raise SystemExit(f'{path}: expected one device target in the bundle, found {targets}')
            subprocess.run([os.path.join(llvm_bin, 'clang-offload-bundler'), '--unbundle', '--type=o',
                            '--targets=' + targets[0], '--input=' + path, '--output=' + co], check=True)
        return subprocess.run([os.path.join(llvm_bin, 'llvm-objdump'), '-d', co], check=True, capture_output=True,
                              text=True).stdout


def vregs(text):
    regs = set()
    for a, b in re.findall(r'\bv\[(\d+):(\d+)\]', text):
        regs |= set(range(int(a), int(b) + 1))
    regs |= {int(a) for a in re.findall(r'\bv(\d+)\b', text)}
    return regs


def sregs(text):
    regs = set()
    for a, b in re.findall(r'\bs\[(\d+):(\d+)\]', text):
        regs |= set(range(int(a), int(b) + 1))
    regs |= {int(a) for a in re.findall(r'\bs(\d+)\b', text)}
    return regs


def functions(disassembly):
    cur, out = None, collections.OrderedDict()
    for line in disassembly.split('\n'):
        m = re.match(r'^[0-9a-f]+ <(.*)>:', line)
        if m:
            cur = m.group(1)
            out[cur] = []
            continue
        if cur is not None and line.startswith('\t'):
            ins = line.strip().split('//')[0].strip()
            if ins:
                out[cur].append(ins)
    return out


def check_ownership(ins_list):
    bad, top = [], -1
    for ins in ins_list:
        regs = vregs(ins)
        if not regs:
            continue
        op, hi = ins.split()[0], max(regs)
        if hi < FIRST_OWNED:
            top = max(top, hi)
            continue
        if op in ASM_OPS:
            continue
        if op == 'v_mov_b32_e32' and re.search(r', 0\s*$', ins) and min(regs) >= ACC_FIRST:
            continue
        if op.startswith(('v_writelane', 'v_readlane')) and regs <= set(SPILL_LANES):
            continue
        bad.append(ins)
    return top, bad


def is_valu(op):
    return op.startswith('v_') and not op.startswith(('v_readfirstlane', 'v_readlane', 'v_cmp'))


def check_wait_states(ins_list):
    bad = []
    for i, ins in enumerate(ins_list):
        op = ins.split()[0]
        if op.startswith(('v_readfirstlane', 'v_readlane')):
            dst, ws = sregs(ins.split(',')[0]), 0
            for nxt in ins_list[i + 1:i + 12]:
                o = nxt.split()[0]
                if o.startswith(('buffer_', 'global_', 'flat_', 'scratch_')) and dst & sregs(nxt) and ws < 5:
                    bad.append(f'{ins}  ->  {nxt}  ({ws} wait states)')
                ws += int(nxt.split()[1]) + 1 if o == 's_nop' else 1
                if ws >= 5:
                    break
        if is_valu(op) and i + 1 < len(ins_list):
            nxt = ins_list[i + 1]
            if nxt.split()[0].startswith(('v_readfirstlane', 'v_readlane')):
                if vregs(ins.split(',')[0]) & vregs(nxt.split(',', 1)[1]):
                    bad.append(f'{ins}  ->  {nxt}  (0 wait states)')
    return bad


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('path')
    ap.add_argument('--llvm-bin', default='/opt/rocm/llvm/bin')
    ap.add_argument('--kernel', default='spmm_rows_kernel', help='substring of the mangled names to check')
    args = ap.parse_args()
    funcs = {k: v for k, v in functions(disassemble(args.path, args.llvm_bin)).items() if args.kernel in k}
    if not funcs:
        print(f'{args.path}: no function matching {args.kernel!r}', file=sys.stderr)
        return 1
    failed = False
    for name, ins_list in funcs.items():
        top, owned = check_ownership(ins_list)
        waits = check_wait_states(ins_list)
        print(f'{name[:72]}: {len(ins_list)} instructions, compiler registers up to v{top}, '
              f'{len(owned)} on owned registers, {len(waits)} short of wait states')
        for ins in owned[:12]:
            print('    owned register touched:', ins)
        for w in waits[:12]:
            print('    wait states:', w)
        failed |= bool(owned) or bool(waits)
    return 1 if failed else 0


if __name__ == '__main__':
    sys.exit(main())
