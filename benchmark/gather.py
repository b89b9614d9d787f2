"""Times gather_coo / gather_csr against index_select and torch.gather on the same row
structures as scatter_segment.py; methodology and table of the reference's
benchmark/gather.py (:62-119).

  python benchmark/gather.py [--with_backward] [--scale 0.25] [--mat ldoor.mat ...] [--json out.json]
"""
import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from benchmark.matrices import print_table, structures, timed  # noqa: E402
from pytorch_scatter_amd import gather_coo, gather_csr  # noqa: E402

WIDTHS = [1, 16, 32, 64, 128, 256, 512]


def check(m, widths, device):
    with torch.no_grad():
        for k in widths:
            x = torch.randn((m.rows, k), device=device)
            want = x.index_select(0, m.row)
            assert torch.equal(want, gather_coo(x, m.row)), (m.label, k, 'gather_coo')
            assert torch.equal(want, gather_csr(x, m.rowptr)), (m.label, k, 'gather_csr')


def methods(m):
    return [
        ('SELECT', lambda x: x.index_select(0, m.row)),
        ('GAT', lambda x: x.gather(0, m.row.view(-1, 1).expand(-1, x.size(1)))),
        ('GAT_COO', lambda x: gather_coo(x, m.row)),
        ('GAT_CSR', lambda x: gather_csr(x, m.rowptr)),
    ]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--with_backward', action='store_true')
    ap.add_argument('--device', default='cuda')
    ap.add_argument('--scale', type=float, default=1.0)
    ap.add_argument('--only', nargs='*')
    ap.add_argument('--mat', nargs='*')
    ap.add_argument('--json')
    ap.add_argument('--plain', action='store_true')
    ap.add_argument('--no-check', action='store_true')
    args = ap.parse_args()

    on_gpu = args.device != 'cpu'
    iters = 20 if on_gpu else 1
    widths = WIDTHS if on_gpu else WIDTHS[:3]
    for _ in range(10):
        torch.randn(100, 100, device=args.device).sum()

    record = {'with_backward': args.with_backward, 'iters': iters, 'widths': widths, 'matrices': {}}
    for m in structures(args):
        if not args.no_check:
            check(m, widths, args.device)
        cells = {label: [] for label, _ in methods(m)}
        for k in widths:
            x = torch.randn((m.rows, k), device=args.device)
            for label, fn in methods(m):
                cells[label].append(timed(fn, x, iters, args.with_backward))
            del x
        print_table(f'{m.label} (avg row length: {m.avg_row_len:.2f}):', widths, list(cells.items()), args.plain)
        record['matrices'][m.label] = {'rows': m.rows, 'entries': m.entries, 'seconds': cells}
        sys.stdout.flush()
    if args.json:
        with open(args.json, 'w') as f:
            json.dump(record, f, indent=1)


if __name__ == '__main__':
    main()
