"""Einsum strings of multi-head attention for inputs of any rank.

The reference takes them from Keras (`_build_proj_equation`, `_build_attention_equation`, imported at reference
src/hgq/layers/attn/mha.py:10) and `_get_output_shape` (mha.py:20-22).  Keras is not a dependency here, so the same
letter assignment is produced by the three functions below: axis 0 is the batch, the last projected axes are
(heads, channels), the attended axes of the key side get fresh letters after the query's."""

from __future__ import annotations

import string

_LETTERS = string.ascii_lowercase


def proj_equation(free_dims: int, bound_dims: int, output_dims: int):
    """``(equation, bias_axes, output_rank)`` of a projection ``[free..., bound...] x [bound..., out...] -> [free..., out...]``."""
    free = _LETTERS[:free_dims]
    bound = _LETTERS[free_dims:free_dims + bound_dims]
    out = _LETTERS[free_dims + bound_dims:free_dims + bound_dims + output_dims]
    return f'{free}{bound},{bound}{out}->{free}{out}', out, free_dims + output_dims


def attention_equations(rank: int, attn_axes):
    """``(dot_product_equation, combine_equation, scores_rank)`` for projected tensors of ``rank`` axes
    ``[batch, seq..., heads, channels]`` attending over ``attn_axes``.

    Scores are laid out ``[batch axes..., query attended axes..., key attended axes...]`` where the batch axes are all
    axes that are neither attended nor the channel axis (so the heads axis is one of them)."""
    attn_axes = tuple(attn_axes)
    query = _LETTERS[:rank]
    kept = [i for i in range(rank) if i not in attn_axes and i != rank - 1]
    key, fresh = '', rank
    for i in range(rank):
        if i in kept or i == rank - 1:
            key += query[i]
        else:
            key += _LETTERS[fresh]
            fresh += 1
    scores = ''.join(query[i] for i in kept) + ''.join(query[i] for i in attn_axes) + ''.join(key[i] for i in attn_axes)
    return f'{key},{query}->{scores}', f'{scores},{key}->{query}', len(scores)


def projected_shape(output_rank: int, known_last_dims, input_shape):
    """Output shape (without the batch axis) of a projection: the input's leading axes, then the known last ones."""
    n = output_rank - len(known_last_dims)
    return list(input_shape[1:n + 1]) + list(known_last_dims)
