"""Command line style of operator creation (README.md:75-77):

    python -m autort --ir "sigmoid_f32[N] = 1 - 1 / (1 + data[N].call(strs.exp))" -i data=float32[N:4096000] -c "tune:5"

parses and lowers the program, compiles its kernels for gfx950 (no GPU needed
for that) and writes the operator's module file, after which
``autort.ops.<name>`` finds it in any later session.
"""
from __future__ import annotations

import argparse
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog='autort', description='Create a persistent custom operator from einstein_v2 text.')
    ap.add_argument('--ir', required=True, help='the program, statements separated by ";" or newlines')
    ap.add_argument('-i', '--input', action='append', default=[], metavar='NAME=DTYPE[DIMS]',
                    help='one input tensor declaration; repeat in calling order')
    ap.add_argument('-c', '--config', default=None, help='e.g. "tune:5" or "~N~:[1,256,1]"')
    ap.add_argument('-n', '--name', default=None, help='operator name (default: name of the last output tensor)')
    ap.add_argument('-e', '--extra-output', action='append', default=[], help='intermediate tensor to return as an output too')
    ap.add_argument('--no-compile', action='store_true', help='write the module file without building the kernels')
    args = ap.parse_args(argv)
    from . import export
    from . import store
    try:
        op = export(ir=args.ir, inputs=args.input, config=args.config, name=args.name, extra_outputs=args.extra_output)
        if not args.no_compile and op.fast_path is None:
            op.compile()
    except Exception as e:       # a usage error, not a crash: report it the way a CLI does
        print(f'autort: {type(e).__name__}: {e}', file=sys.stderr)
        return 1
    how = 'hand-written kernel' if op.fast_path is not None else f'{len(op.plans)} generated kernel(s)'
    print(f'Module file for operator `{op.name}` has been exported to `{store.module_path(op.name)}` ({how}).')
    return 0


if __name__ == '__main__':
    sys.exit(main())
