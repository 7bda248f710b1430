"""Which kernels of the library a traced run launched.

    python3 tests/kernel_coverage.py <kernel_stats.csv> [<kernel_stats.csv> ...]

The CSV files are the per-kernel statistics that `rocprofv3 --kernel-trace --stats --output-format csv` writes for a run
(of the GPU tests, say).  The library holds one host stub per compiled kernel (`nm -C` shows them as
`tk::__device_stub__<kernel>(arguments)`); every template instantiation is a kernel of its own.  Prints, per kernel
family, how many kernels are compiled and how many of them the run launched, then the ones it never launched; the exit
status is 1 if there are any."""
import collections
import csv
import os
import re
import subprocess
import sys

LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), 'tilekernels_amd', 'lib', 'libtk_quant.so')


def compiled_kernels(lib: str) -> list:
    out = subprocess.run(['nm', '-C', lib], check=True, capture_output=True, text=True).stdout
    names = {re.sub(r'\(.*$', '', line.split('__device_stub__', 1)[1]).strip() for line in out.splitlines() if '__device_stub__' in line}
    return sorted(names)


def launched_kernels(paths) -> dict:
    calls = collections.Counter()
    for path in paths:
        with open(path, newline='') as f:
            for row in csv.DictReader(f):
                if 'tk::' in row['Name']:
                    calls[re.sub(r'\(.*$', '', row['Name'].split('tk::', 1)[1]).strip()] += int(row['Calls'])
    return calls


def main(argv) -> int:
    if len(argv) < 2:
        print(__doc__)
        return 2
    squeeze = lambda s: re.sub(r'\s+', '', s).replace('tk::', '')
    launched = {squeeze(k): v for k, v in launched_kernels(argv[1:]).items()}
    compiled = compiled_kernels(LIB)
    family = lambda k: k.split('<')[0]
    per_family = collections.defaultdict(lambda: [0, 0, 0])
    missing = []
    for k in compiled:
        n = launched.get(squeeze(k), 0)
        row = per_family[family(k)]
        row[0] += 1
        row[1] += 1 if n else 0
        row[2] += n
        if not n:
            missing.append(k)
    for fam in sorted(per_family):
        c, l, n = per_family[fam]
        print(f'  {fam:34s} {c:4d} compiled   {l:4d} launched   {n:7d} launches')
    print(f'  {"total":34s} {len(compiled):4d} compiled   {len(compiled) - len(missing):4d} launched   {sum(r[2] for r in per_family.values()):7d} launches')
    for k in missing:
        print('never launched:', k)
    return 1 if missing else 0


if __name__ == '__main__':
    sys.exit(main(sys.argv))
