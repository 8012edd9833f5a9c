# Derived from opveclib/examples/conv1D.py of opveclib (https://github.com/opveclib/opveclib),
# Copyright 2016 Hewlett Packard Enterprise Development LP, licensed under the Apache License, Version 2.0;
# see the NOTICE file at the root of this repository.  The operator's statements are that file's (they define the
# result); docstrings, argument checks and everything around them are new.
"""
One-dimensional multi-channel convolution / cross-correlation written against the DSL, with worker-local tensors
(the reference's opveclib/examples/conv1D.py:17-207 computes the same function with a ring buffer per worker).

A worker owns ELEMENTS_PER_WORKER consecutive output elements of one (batch, filter) pair.  Per input channel it
copies the filter taps and the stretch of input it needs (zero outside the signal) into local tensors, then
accumulates products in float64, channel by channel and tap by tap in ascending order - the order of the
reference's loops, so both produce the same sums.
"""
from .. import expression as ovl
from ..operator import operator

ELEMENTS_PER_WORKER = 10


def output_geometry(num_elements, filter_size, mode):
    """(index of the input element under tap 0 of output element 0, number of output elements) per border mode."""
    left_apron = filter_size // 2
    right_apron = filter_size - left_apron - 1
    if mode in ('same', 'valid') and filter_size > num_elements:
        raise ValueError('filter size, ' + str(filter_size) + ',  cannot be larger than number of elements, ' +
                         str(num_elements))
    if mode == 'same':
        return -left_apron, num_elements
    if mode == 'valid':
        return 0, num_elements - (left_apron + right_apron)
    if mode == 'full':
        return -(filter_size - 1), num_elements + filter_size - 1
    raise ValueError("mode must be 'same', 'valid', or 'full'.")


@operator()
def conv_1d(x, v, kernel_orientation='as-is', stride=1, mode='same', data_format='NCE'):
    """
    :param x: input of rank 3; ``data_format`` names its axes: N batches, C channels, E elements
    :param v: filters with the same axis order: N filters, C channels, E taps
    :param kernel_orientation: 'as-is' (cross-correlation) or 'flipped' (convolution)
    :param stride: must be 1 (the reference validates this argument and then computes with stride 1)
    :param mode: 'same', 'valid' or 'full'
    :return: output with N batches, C = number of filters, E output elements, in ``data_format`` order, dtype of x
    """
    if kernel_orientation not in ('as-is', 'flipped'):
        raise ValueError("kernel_orientation must be 'as-is' or 'flipped'")
    if x.rank != 3 or v.rank != 3 or sorted(data_format) != ['C', 'E', 'N']:
        raise ValueError('x and v must have rank 3 and data_format must be a permutation of "NCE"')
    n_axis, c_axis, e_axis = (data_format.find(k) for k in 'NCE')
    num_batches, num_channels, num_elements = x.shape[n_axis], x.shape[c_axis], x.shape[e_axis]
    num_filters, filter_size = v.shape[n_axis], v.shape[e_axis]
    if num_channels != v.shape[c_axis]:
        raise ValueError('Channel axis size of input must match that of the filter.')
    if not isinstance(stride, int) or stride != 1:
        raise ValueError('Only stride 1 is supported')
    first_input, output_elements = output_geometry(num_elements, filter_size, mode)

    def at(n, c, e):
        index = [None, None, None]
        index[n_axis], index[c_axis], index[e_axis] = n, c, e
        return index

    out_shape = at(num_batches, num_filters, output_elements)
    out = ovl.output(out_shape, x.dtype)

    per_worker = ELEMENTS_PER_WORKER
    element_workers = (output_elements + per_worker - 1) // per_worker
    pos = ovl.position_in([num_batches, num_filters, element_workers])
    batch, cur_filter, block = pos[0], pos[1], pos[2]
    first_out = ovl.cast(block, ovl.int64) * per_worker
    block_elements = ovl.variable(per_worker, ovl.int64)
    if output_elements % per_worker:
        with ovl.if_(block == element_workers - 1):
            block_elements <<= output_elements % per_worker

    span = filter_size + per_worker - 1
    taps = ovl.zeros((filter_size,), v.dtype)
    window = ovl.zeros((span,), x.dtype)
    accum = ovl.zeros((per_worker,), ovl.float64)

    for channel in ovl.arange(num_channels):
        for k in ovl.arange(filter_size):
            source = k if kernel_orientation == 'as-is' else (filter_size - 1) - k
            taps[k] = v[at(cur_filter, channel, source)]
        for w in ovl.arange(span):
            e = first_out + w + first_input
            inside = ovl.logical_and(e >= 0, e < num_elements)
            with ovl.if_(inside):
                window[w] = x[at(batch, channel, e)]
            with ovl.else_():
                window[w] = 0
        for i in ovl.arange(block_elements):
            for k in ovl.arange(filter_size):
                accum[i] = accum[i] + ovl.cast(window[i + k], ovl.float64) * ovl.cast(taps[k], ovl.float64)

    for i in ovl.arange(block_elements):
        out[at(batch, cur_filter, first_out + i)] = ovl.cast(accum[i], x.dtype)
    return out
