"""Persisted operators: one ``<name>.mod`` text file per exported operator.

The reference's wheel keeps every exported operator as a module file under
``./ops`` so that ``autort.ops.<name>`` works in later sessions and from the
command line (README.md:75-86,139-141; the legacy tree writes the same kind of
record as ``my_kernel.cc`` + a tuning database, antares/antares_compiler.py:679-688).
Here a module file holds what is needed to rebuild the operator — the IR, the
input declarations, the config (including what a tuning run chose) — followed by
the generated kernel container, which is informational: code objects are
recompiled from it on demand and cached by content hash.

Directory: ``$AUTORT_OPS_DIR`` if set, else ``antares_amd/_ops`` next to the package.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

FORMAT = 'autort-amd-module-1'
_HEADER_END = '// ---- kernels (informational) ----'


def ops_dir() -> str:
    d = os.environ.get('AUTORT_OPS_DIR')
    if not d:
        d = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), '_ops')
    return d


def module_path(name: str) -> str:
    if not name or any(c in name for c in '/\\\0') or name.startswith('.'):
        raise ValueError(f'`{name}` is not a usable operator name')
    return os.path.join(ops_dir(), name + '.mod')


def save(name: str, ir: str, inputs: List[str], config: Optional[str], extra_outputs: List[str],
         tuned: Optional[Dict[str, object]] = None, source: str = '') -> str:
    """Writes (atomically) the module file of an operator and returns its path."""
    record = {'format': FORMAT, 'name': name, 'ir': ir, 'inputs': list(inputs), 'config': config,
              'extra_outputs': list(extra_outputs), 'tuned': tuned or {}}
    path = module_path(name)
    os.makedirs(os.path.dirname(path), exist_ok=True)
    tmp = f'{path}.{os.getpid()}.tmp'
    with open(tmp, 'w') as f:
        f.write('// MODULE: ' + json.dumps(record, sort_keys=True) + '\n')
        f.write(_HEADER_END + '\n')
        f.write(source)
    os.replace(tmp, path)
    return path


def load(name: str) -> Optional[Dict[str, object]]:
    """The record of a persisted operator, or None if there is none."""
    try:
        path = module_path(name)
    except ValueError:
        return None
    if not os.path.isfile(path):
        return None
    with open(path) as f:
        first = f.readline()
    if not first.startswith('// MODULE: '):
        raise ValueError(f'{path} is not an operator module file')
    record = json.loads(first[len('// MODULE: '):])
    if record.get('format') != FORMAT:
        raise ValueError(f'{path}: unknown module format {record.get("format")!r}')
    return record


def names() -> List[str]:
    d = ops_dir()
    if not os.path.isdir(d):
        return []
    return sorted(f[:-4] for f in os.listdir(d) if f.endswith('.mod'))
