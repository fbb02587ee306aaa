"""Writes parser_golden.json: what the reference's own parser (lang/einstein_v2.py) makes of every worked
program in tests/ir_examples.py - per statement the output name, the dtype of the r-value, data and reduce axes
with their inferred ranges, the reduce type, and the expression printed back by the reference's reverse emitter
(emit_antares_ir, lang/einstein_v2.py:419-485).

Run in the build container only (the reference tree lives at /root/reference and does not travel):

    python tests/golden/make_parser_golden.py

The statement loop below is the first half of ir_graph_parser (lang/einstein_v2.py:519-555); its second half
(the pass pipeline, a no-op in the reference: lang/pass/200_simplify.py:41-42) is not run.
"""
import copy
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, '/root/reference')

sys.path.insert(0, HERE)
from ir_examples import EXAMPLES          # noqa: E402
from parser_corner_cases import CORNER_CASES, inputs_for   # noqa: E402
from lang import einstein_v2 as ref      # noqa: E402


def main():
    out = {}
    programs = {name: (program, input_dict) for name, (program, input_dict, _, _) in EXAMPLES.items()}
    for name, statement in CORNER_CASES.items():
        programs['corner/' + name] = (statement, inputs_for(statement))
    for name, (program, input_dict) in programs.items():
        ref.full_tensor_dict = copy.deepcopy(input_dict)
        ref.vamap_tensor = {key: [int(d) for d in input_dict[key]['shape']] for key in input_dict}
        records = []
        for text in [s.strip() for s in program.split(';')]:
            if not text:
                continue
            ref.explicit_range = None
            try:
                ast = ref.parse_to_ast(text)
            except Exception as e:       # the reference rejects the statement: record that it does
                records.append({'statement': text, 'error': type(e).__name__})
                break
            props = ast['props']
            k = props['output_name']
            ref.full_tensor_dict[k] = {'shape': [x['range'] for x in props['data_axes']], 'dtype': ast['root']._dtype}
            ref.vamap_tensor[k] = [ref.explicit_range[x['name']][0] for x in props['data_axes']]
            try:
                printed = ref.emit_antares_ir(ast)
            except Exception:            # the reverse emitter has no case for one-operand operators (:437-440)
                printed = None
            records.append({
                'statement': text,
                'output': k,
                'dtype': ast['root']._dtype,
                'data_axes': [[x['name'], x['range']] for x in props['data_axes']],
                'reduce_axes': [[x['name'], x['range']] for x in props['reduce_axes']],
                'reduce_type': props['reduce_type'],
                'inputs': sorted(props['input_dict']),
                'ir': printed,
            })
        out[name] = records
    path = os.path.join(HERE, 'parser_golden.json')
    with open(path, 'w') as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print('wrote', path, len(out), 'programs,', sum(len(v) for v in out.values()), 'statements')


if __name__ == '__main__':
    main()
