"""``python -m autort.utils.export -s STEPS`` (README.md:139-141): tunes `gemm_f32` for up to STEPS launch
configurations on this device and writes its module file, which `autort.ops.gemm_f32` (and
``autort.utils.mmtest``) pick up in later sessions."""
from __future__ import annotations

import argparse
import sys

from . import GEMM_F32_INPUTS


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog='autort.utils.export')
    ap.add_argument('-s', '--steps', type=int, default=20, help='launch configurations to time at most')
    ap.add_argument('--size', type=int, default=4096)
    args = ap.parse_args(argv)
    import torch
    from .. import store
    from .mmtest import gemm_f32_op
    op = gemm_f32_op(config=f'tune:{max(1, args.steps)}')
    n = args.size
    dev = torch.device('cuda')
    op(torch.randn(n, n, device=dev), torch.randn(n, n, device=dev))          # the first call per shape runs the search
    torch.cuda.synchronize()
    print(f'\n  Module file for operator `{op.name}` has been exported to `{store.module_path(op.name)}`.\n', flush=True)
    assert GEMM_F32_INPUTS and op.tuned, 'no launch configuration was recorded'
    return 0


if __name__ == '__main__':
    sys.exit(main())
