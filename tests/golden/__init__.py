"""Loader of the known-answer fixtures in this directory (data taken from the reference's documentation and tests)."""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def _numbers(values, dtype):
    def one(v):
        if isinstance(v, str):
            return float(v) if v in ('inf', '-inf', 'nan') else float.fromhex(v)
        return v
    if values and isinstance(values[0], list):
        return np.array([[one(v) for v in row] for row in values], dtype=dtype)
    return np.array([one(v) for v in values], dtype=dtype)


def known_answers():
    """[(name, operator outputs to evaluate, expected array or None, expected sum or None, absolute tolerance)]"""
    from opveclib_amd.examples import shift_cyclic, cumsum, cumprod, expm1, log1p, graph
    with open(os.path.join(HERE, 'known_answers.json')) as f:
        vectors = json.load(f)['vectors']
    cases = []
    for v in vectors:
        dtype = np.dtype(v['dtype'])
        if v['operator'] == 'triangles':
            out = graph.triangles_op(*graph.adjacency_from_edges(graph.EXAMPLE_EDGES))
            cases.append((v['name'], out, None, v['expected_sum'], 0.0))
            continue
        x = _numbers(v['input'], dtype)
        build = {'shift_cyclic': lambda a: shift_cyclic(a), 'expm1': lambda a: expm1(a), 'log1p': lambda a: log1p(a),
                 'cumsum': lambda a: cumsum(a, axis=v.get('axis', 0)),
                 'cumprod': lambda a: cumprod(a, axis=v.get('axis', 0))}[v['operator']]
        cases.append((v['name'], build(x), _numbers(v['expected'], dtype), None, float(v.get('atol', 0.0))))
    return cases
