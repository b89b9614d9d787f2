"""Times scatter / segment_coo / segment_csr against PyTorch's own scatter_add_ and a dense
reduction of the same volume, per feature width, on the row structures of four sparse
matrices. Same methodology and table as the reference's benchmark/scatter_segment.py
(:109-210): 20 iterations per cell on the GPU, widths 1..512, the index once in row order
(`_ROW`) and once shuffled (`_COL`), fastest method per column in bold.

  python benchmark/scatter_segment.py --reduce sum [--with_backward] [--scale 0.25]
                                      [--mat ldoor.mat ...] [--json out.json]
"""
import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from benchmark.matrices import print_table, structures, timed  # noqa: E402
from pytorch_scatter_amd import scatter, segment_coo, segment_csr  # noqa: E402

WIDTHS = [1, 16, 32, 64, 128, 256, 512]


def check(m, widths, device):
    """The three operator families must agree on every reduction (benchmark/scatter_segment.py:35-79)."""
    n = m.rows
    with torch.no_grad():
        for k in widths:
            x = torch.randn((m.entries, k), device=device)
            x = x.squeeze(-1) if k == 1 else x
            for reduce in ('sum', 'mean', 'min', 'max'):
                a = scatter(x, m.row, dim=0, dim_size=n, reduce=reduce)
                b = segment_coo(x, m.row, dim_size=n, reduce=reduce)
                c = segment_csr(x, m.rowptr, reduce=reduce)
                assert torch.allclose(a, b, atol=1e-4), (m.label, k, reduce, 'scatter vs segment_coo')
                assert torch.allclose(a, c, atol=1e-4), (m.label, k, reduce, 'scatter vs segment_csr')
            del x


def methods(m, reduce):
    n = m.rows

    def torch_scatter_add(index):
        def run(x):
            out = x.new_zeros(n, *x.shape[1:])
            idx = index.view(-1, 1).expand_as(x) if x.dim() > 1 else index
            return out.scatter_add_(0, idx, x)
        return run

    return [
        ('SCA1_ROW', torch_scatter_add(m.row)),
        ('SCA1_COL', torch_scatter_add(m.row_shuffled)),
        ('SCA2_ROW', lambda x: scatter(x, m.row, dim=0, dim_size=n, reduce=reduce)),
        ('SCA2_COL', lambda x: scatter(x, m.row_shuffled, dim=0, dim_size=n, reduce=reduce)),
        ('SEG_COO', lambda x: segment_coo(x, m.row, reduce=reduce)),
        ('SEG_CSR', lambda x: segment_csr(x, m.rowptr, reduce=reduce)),
    ]


def dense_methods(reduce):
    # a dense tensor of the same volume, reduced over its second-to-last / last dimension
    op = getattr(torch, reduce)
    return [('DENSE1', lambda x: op(x, dim=-2)), ('DENSE2', lambda x: op(x, dim=-1))]


def time_matrix(m, args, widths, iters):
    sparse, dense = methods(m, args.reduce), dense_methods(args.reduce)
    cells = {label: [] for label, _ in sparse + dense}
    per_row = int(m.avg_row_len + 1)
    for k in widths:
        x = torch.randn((m.entries, k), device=args.device)
        x = x.squeeze(-1) if k == 1 else x
        for label, fn in sparse:
            cells[label].append(timed(fn, x, iters, args.with_backward))
        del x
        try:
            x = torch.randn((m.rows, per_row, k), device=args.device)
            cells['DENSE1'].append(timed(dense[0][1], x, iters, args.with_backward))
            x = x.view(m.rows, k, per_row)
            cells['DENSE2'].append(timed(dense[1][1], x, iters, args.with_backward))
            del x
        except RuntimeError as e:
            if 'out of memory' not in str(e):
                raise
            torch.cuda.empty_cache()
            for label in ('DENSE1', 'DENSE2'):
                if len(cells[label]) < len(cells['SEG_CSR']):
                    cells[label].append(float('inf'))
    return cells


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--reduce', required=True, choices=['sum', 'mean', 'min', 'max'])
    ap.add_argument('--with_backward', action='store_true')
    ap.add_argument('--device', default='cuda')
    ap.add_argument('--scale', type=float, default=1.0, help='shrink the synthetic matrices')
    ap.add_argument('--only', nargs='*', help='matrix names to run (default: all four)')
    ap.add_argument('--mat', nargs='*', help='SuiteSparse .mat files to use instead of the synthetic structures')
    ap.add_argument('--json', help='also write the timings to this file')
    ap.add_argument('--plain', action='store_true', help='no terminal escapes in the tables')
    ap.add_argument('--no-check', action='store_true')
    args = ap.parse_args()

    on_gpu = args.device != 'cpu'
    iters = 20 if on_gpu else 1
    widths = WIDTHS if on_gpu else WIDTHS[:3]
    for _ in range(10):   # warm-up of the device and the allocator
        torch.randn(100, 100, device=args.device).sum()

    record = {'reduce': args.reduce, 'with_backward': args.with_backward, 'iters': iters, 'widths': widths,
              'unit': 'seconds per %d calls' % iters, 'matrices': {}}
    for m in structures(args):
        if not args.no_check:
            check(m, widths, args.device)
        cells = time_matrix(m, args, widths, iters)
        print_table(f'{m.label} (avg row length: {m.avg_row_len:.2f}):', widths, list(cells.items()), args.plain)
        record['matrices'][m.label] = {'rows': m.rows, 'entries': m.entries, 'seconds': cells}
        sys.stdout.flush()
    if args.json:
        with open(args.json, 'w') as f:
            json.dump(record, f, indent=1)


if __name__ == '__main__':
    main()
