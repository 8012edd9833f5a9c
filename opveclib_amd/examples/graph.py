# Derived from opveclib/examples/test_graph.py of opveclib (https://github.com/opveclib/opveclib),
# Copyright 2016 Hewlett Packard Enterprise Development LP, licensed under the Apache License, Version 2.0;
# see the NOTICE file at the root of this repository.  The operator's statements are that file's (they define the
# result); docstrings, argument checks and everything around them are new.
"""
Triangle counting on an undirected graph with one worker per edge (the edge-iterator strategy of the reference's
opveclib/examples/test_graph.py:17-92): a worker on edge (u, v), u > v, merges the sorted neighbour lists of u and v
and counts the common neighbours smaller than v, so each triangle is counted exactly once.

The graph is held as a compressed adjacency list: ``start_edge[k] .. start_edge[k+1]`` delimit vertex k's slice of
``to_vertex`` (neighbours with a smaller index, ascending), ``from_vertex`` repeats the owning vertex per edge.
The merge needs a data-dependent number of steps; the DSL has counted loops only, so the loop runs for the largest
number of steps the two lists allow and idles once one list is exhausted (as the reference does).  Neighbour reads
past a list's end are clamped to the last edge instead of reading beyond the array.
"""
import numpy as np

from .. import expression as ovl
from ..operator import operator, evaluate

# the reference's example graph: 7 vertices, 20 directed edge records (10 undirected edges), 3 triangles
# (opveclib/examples/test_graph.py:183-202, 130)
EXAMPLE_EDGES = [(0, 1), (1, 2), (2, 3), (3, 4), (4, 5), (5, 6), (0, 6), (1, 3), (3, 5), (1, 6),
                 (1, 0), (2, 1), (3, 2), (4, 3), (5, 4), (6, 5), (6, 0), (3, 1), (5, 3), (6, 1)]
EXAMPLE_TRIANGLES = 3


@operator()
def triangles_op(start_edge, from_vertex, to_vertex):
    """:return: uint64 tensor with the number of triangles closed by every edge."""
    num_edges = to_vertex.shape[0]
    edge = ovl.position_in(to_vertex.shape)[0]
    count = ovl.output(to_vertex.shape, ovl.uint64)
    found = ovl.variable(0, ovl.uint64)
    last = num_edges - 1

    u = ovl.variable(from_vertex[edge], from_vertex.dtype)
    v = ovl.variable(to_vertex[edge], to_vertex.dtype)
    u_at = ovl.variable(start_edge[u], start_edge.dtype)
    u_end = ovl.variable(start_edge[u + 1], start_edge.dtype)
    v_at = ovl.variable(start_edge[v], start_edge.dtype)
    v_end = ovl.variable(start_edge[v + 1], start_edge.dtype)
    u_next = ovl.variable(to_vertex[ovl.minimum(u_at, last)], to_vertex.dtype)
    v_next = ovl.variable(to_vertex[ovl.minimum(v_at, last)], to_vertex.dtype)

    for _ in ovl.arange((u_end - u_at) + (v_end - v_at)):
        merging = ovl.logical_and(ovl.logical_and(u_at < u_end, v_at < v_end), u_next < v)
        with ovl.if_(merging):
            with ovl.if_(u_next < v_next):
                u_at <<= u_at + 1
                u_next <<= to_vertex[ovl.minimum(u_at, last)]
            with ovl.elif_(u_next > v_next):
                v_at <<= v_at + 1
                v_next <<= to_vertex[ovl.minimum(v_at, last)]
            with ovl.else_():
                found <<= found + 1
                u_at <<= u_at + 1
                v_at <<= v_at + 1
                u_next <<= to_vertex[ovl.minimum(u_at, last)]
                v_next <<= to_vertex[ovl.minimum(v_at, last)]

    count[edge] = found
    return count


def triangles(start_edge, from_vertex, to_vertex, target_language='hip'):
    """Total number of triangles of the graph (test_graph.py:95-121)."""
    count = evaluate(triangles_op(start_edge, from_vertex, to_vertex), target_language=target_language)
    if not isinstance(count, np.ndarray):
        count = count.cpu().numpy()
    return int(np.sum(count, axis=0, dtype=np.uint64))


def adjacency_from_edges(edges):
    """
    Compressed adjacency list of an undirected graph given as (a, b) pairs in any order and multiplicity; self loops
    and duplicates are dropped.  Every undirected edge is stored once, under its larger end point.

    :return: (start_edge[num_vertices + 1], from_vertex[num_edges], to_vertex[num_edges]) as uint64 arrays
    """
    pairs = np.asarray(edges, dtype=np.int64).reshape(-1, 2)
    pairs = pairs[pairs[:, 0] != pairs[:, 1]]
    hi = np.maximum(pairs[:, 0], pairs[:, 1])
    lo = np.minimum(pairs[:, 0], pairs[:, 1])
    unique = np.unique(np.stack([hi, lo], axis=1), axis=0)      # sorted by (hi, lo): neighbour lists ascend
    num_vertices = int(pairs.max()) + 1 if pairs.size else 0
    start = np.zeros(num_vertices + 1, dtype=np.uint64)
    np.cumsum(np.bincount(unique[:, 0], minlength=num_vertices), out=start[1:])
    return start, unique[:, 0].astype(np.uint64), unique[:, 1].astype(np.uint64)


def count_triangles_dense(edges):
    """Triangle count from the adjacency matrix, trace(A^3) / 6: an independent check for small graphs."""
    pairs = np.asarray(edges, dtype=np.int64).reshape(-1, 2)
    n = int(pairs.max()) + 1
    a = np.zeros((n, n), dtype=np.int64)
    for p, q in pairs:
        if p != q:
            a[p, q] = a[q, p] = 1
    return int(np.trace(a @ a @ a)) // 6
