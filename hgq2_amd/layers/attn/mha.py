"""QMultiHeadAttention (reference src/hgq/layers/attn/mha.py:27-537): four QEinsumDense projections (query / key /
value with output quantizers, attention_output), scaled dot-product scores, the table softmax, and the EBOPs of the
two score contractions, for inputs ``[batch, seq..., features]`` of any rank attending over all sequence axes.

Rank-3 inputs ``[batch, sequence, features]`` take the one-pass attention kernels.  With more sequence axes the
projections run on the same dense kernels, the two score contractions on the attention contraction kernels over the
flattened sequence axes, and the softmax over its trailing axes stage by stage."""

from __future__ import annotations

import math

import torch

from ... import ops
from ...core import Constant
from ...quantizer import Quantizer
from ...quantizer.config import QuantizerConfig
from ..core.base import QLayerBase
from ..core.einsum_dense import QEinsumDense
from ..softmax import QSoftmax
from ._equations import attention_equations, proj_equation, projected_shape

# with the sequence axes flattened: key [B,S,N,H], query [B,T,N,H] -> scores [B,N,T,S] -> [B,T,N,H]
_DOT_EQ, _COMBINE_EQ = 'aecd,abcd->acbe', 'acbe,aecd->abcd'

FUSED = True  # module switch: False composes scores, softmax and combine from their own kernels (cross-check)


class QMultiHeadAttention(QLayerBase):
    __output_quantizer_handled__ = True

    def __init__(self, num_heads, key_dim, value_dim=None, dropout=0.0, use_bias=True, output_shape=None,
                 attention_axes=None, kernel_initializer='glorot_uniform', bias_initializer='zeros', seed=None,
                 fuse='none', qkvo_iq_conf=None, qkvo_kq_conf=None, qkvo_bq_conf=None, qkvo_oq_conf=None,
                 softmax_iq_conf=None, softmax_exp_iq_conf=None, softmax_exp_oq_conf=None, softmax_inv_iq_conf=None,
                 softmax_inv_oq_conf=None, softmax_oq_conf=None, stable_softmax=True,
                 softmax_allow_heterogeneous_table: bool = False, parallelization_factor=-1, **kwargs):
        super().__init__(**kwargs)
        self._attention_axes = None if attention_axes is None else tuple(
            attention_axes if isinstance(attention_axes, (tuple, list)) else (attention_axes,))
        self._num_heads, self._key_dim = int(num_heads), int(key_dim)
        self._value_dim = int(value_dim) if value_dim else int(key_dim)
        self._dropout, self._use_bias, self._output_shape = float(dropout), use_bias, output_shape
        self._kernel_initializer, self._bias_initializer = kernel_initializer, bias_initializer
        self._qkvo_iq_conf = qkvo_iq_conf or QuantizerConfig(place='datalane')
        self._qkvo_kq_conf = qkvo_kq_conf or QuantizerConfig(place='weight')
        self._qkvo_bq_conf = qkvo_bq_conf or QuantizerConfig(place='bias')
        self._qkvo_oq_conf = qkvo_oq_conf or QuantizerConfig(place='datalane')
        self._softmax_iq_conf = softmax_iq_conf or QuantizerConfig(place='datalane')
        self._softmax_exp_iq_conf = softmax_exp_iq_conf or QuantizerConfig(place='datalane', overflow_mode='SAT')
        self._softmax_exp_oq_conf = softmax_exp_oq_conf or QuantizerConfig(place='table')
        self._softmax_inv_iq_conf = softmax_inv_iq_conf or QuantizerConfig(place='datalane')
        self._softmax_inv_oq_conf = softmax_inv_oq_conf or QuantizerConfig(place='table')
        self._softmax_oq_conf = softmax_oq_conf or QuantizerConfig(place='datalane')
        self._softmax_allow_heterogeneous_table = softmax_allow_heterogeneous_table
        self.parallelization_factor = parallelization_factor
        self._stable_softmax = stable_softmax
        self._fuse = fuse.lower()
        self._inverse_sqrt_key_dim = 1.0 / math.sqrt(float(key_dim))

    def get_config(self):
        config = super().get_config()
        config.pop('oq_conf', None)
        config.update({'num_heads': self._num_heads, 'key_dim': self._key_dim, 'value_dim': self._value_dim, 'dropout': self._dropout,
                       'attention_axes': self._attention_axes,
                       'use_bias': self._use_bias, 'output_shape': self._output_shape, 'kernel_initializer': self._kernel_initializer,
                       'bias_initializer': self._bias_initializer, 'fuse': self._fuse, 'qkvo_iq_conf': self._qkvo_iq_conf,
                       'qkvo_kq_conf': self._qkvo_kq_conf, 'qkvo_bq_conf': self._qkvo_bq_conf, 'qkvo_oq_conf': self._qkvo_oq_conf,
                       'softmax_iq_conf': self._softmax_iq_conf, 'softmax_exp_iq_conf': self._softmax_exp_iq_conf,
                       'softmax_exp_oq_conf': self._softmax_exp_oq_conf, 'softmax_inv_iq_conf': self._softmax_inv_iq_conf,
                       'softmax_inv_oq_conf': self._softmax_inv_oq_conf, 'softmax_oq_conf': self._softmax_oq_conf,
                       'stable_softmax': self._stable_softmax,
                       'softmax_allow_heterogeneous_table': self._softmax_allow_heterogeneous_table,
                       'parallelization_factor': self.parallelization_factor})
        return config

    def _sub_kwargs(self):
        return dict(kernel_initializer=self._kernel_initializer, bias_initializer=self._bias_initializer,
                    iq_conf=self._qkvo_iq_conf.copy(), kq_conf=self._qkvo_kq_conf.copy(), bq_conf=self._qkvo_bq_conf.copy(),
                    oq_conf=self._qkvo_oq_conf.copy(), enable_ebops=self.enable_ebops, beta0=self._beta0.clone(),
                    parallelization_factor=self.parallelization_factor)

    def _build_sub(self, layer, shape):
        layer._build_device = self._build_device
        layer.build(tuple(shape))
        layer.built = True

    def build(self, query_shape, value_shape=None, key_shape=None):
        if isinstance(query_shape, list) and query_shape and isinstance(query_shape[0], (tuple, list)):
            shapes = list(query_shape)
            query_shape = shapes[0]
            value_shape = shapes[1] if len(shapes) > 1 else None
            key_shape = shapes[2] if len(shapes) > 2 else None
        value_shape = query_shape if value_shape is None else value_shape
        key_shape = value_shape if key_shape is None else key_shape
        if len(query_shape) < 3 or len(value_shape) != len(query_shape) or len(key_shape) != len(query_shape):
            raise ValueError('QMultiHeadAttention: query, value and key must be [batch, seq..., features] of one rank')
        if self._fuse == 'qkv':
            assert query_shape == value_shape == key_shape, 'For fuse=qkv, query, key and value must have the same shape'
        if self._fuse == 'kv':
            assert value_shape == key_shape, 'For fuse=kv, key and value must have the same shape'
        if tuple(value_shape[1:-1]) != tuple(key_shape[1:-1]):
            raise ValueError('All dimensions of `value` and `key`, except the last one, must be equal.')
        rank = len(query_shape)
        N = self._num_heads
        eq, bias_axes, out_rank = proj_equation(rank - 1, 1, 2)
        bias = bias_axes if self._use_bias else None
        self._query_dense = QEinsumDense(eq, output_shape=projected_shape(out_rank - 1, [N, self._key_dim], query_shape),
                                         bias_axes=bias, name='query', enable_iq=self.enable_iq and not self._fuse == 'qkv',
                                         enable_oq=True, **self._sub_kwargs())
        self._key_dense = QEinsumDense(eq, output_shape=projected_shape(out_rank - 1, [N, self._key_dim], key_shape),
                                       bias_axes=None, name='key', enable_iq=self.enable_iq and self._fuse not in ('qkv', 'kv'),
                                       enable_oq=True, **self._sub_kwargs())
        self._value_dense = QEinsumDense(eq, output_shape=projected_shape(out_rank - 1, [N, self._value_dim], value_shape),
                                         bias_axes=bias, name='value', enable_iq=self.enable_iq, enable_oq=True, **self._sub_kwargs())
        self._build_sub(self._value_dense, value_shape)
        if self._fuse == 'qkv' and self.enable_iq:
            self._query_dense._iq = self._value_dense._iq
            self._query_dense._enable_iq = True
        if self._fuse in ('qkv', 'kv') and self.enable_iq:
            self._key_dense._iq = self._value_dense._iq
            self._key_dense._enable_iq = True
        self._build_sub(self._query_dense, query_shape)
        self._build_sub(self._key_dense, key_shape)

        # the reference sizes the softmax as [batch, heads, query seq..., key seq...] (mha.py:352-355), which is the
        # layout of the scores only when every sequence axis is attended: that is the case built here
        all_axes = tuple(range(1, out_rank - 2))
        if self._attention_axes is None:
            self._attention_axes = all_axes
        if tuple(a % out_rank for a in self._attention_axes) != all_axes:
            raise NotImplementedError('QMultiHeadAttention: attention over a subset of the sequence axes is not supported')
        self._dot_eq, self._combine_eq, scores_rank = attention_equations(out_rank, self._attention_axes)
        q_seq, k_seq = tuple(query_shape[1:-1]), tuple(value_shape[1:-1])
        self._n_seq = len(q_seq)
        self._T, self._S = math.prod(q_seq), math.prod(k_seq)
        norm_axes = tuple(range(scores_rank - len(self._attention_axes), scores_rank))
        self._softmax = QSoftmax(
            enable_oq=True, axis=norm_axes, stable=self._stable_softmax, iq_conf=self._softmax_iq_conf,
            exp_iq_conf=self._softmax_exp_iq_conf, exp_oq_conf=self._softmax_exp_oq_conf,
            inv_iq_conf=self._softmax_inv_iq_conf, inv_oq_conf=self._softmax_inv_oq_conf, oq_conf=self._softmax_oq_conf,
            allow_heterogeneous_table=self._softmax_allow_heterogeneous_table, input_scaler=self._inverse_sqrt_key_dim,
            enable_ebops=self.enable_ebops, name=f'{self.name}_softmax')  # a fixed name: variable paths must be reproducible
        self._inverse_sqrt_key_dim = 1.0  # the scale now lives in the softmax's exp table
        self._scores_shape = (query_shape[0], N) + q_seq + k_seq
        self._build_sub(self._softmax, self._scores_shape)

        out_shape = self._output_shape if self._output_shape else [query_shape[-1]]
        if not isinstance(out_shape, (tuple, list)):
            out_shape = [out_shape]
        o_eq, o_bias, o_rank = proj_equation(rank - 1, 2, len(out_shape))
        self._output_dense = QEinsumDense(o_eq, output_shape=projected_shape(o_rank - 1, out_shape, query_shape),
                                          bias_axes=o_bias if self._use_bias else None, name='attention_output', enable_iq=True,
                                          enable_oq=self.enable_oq, **self._sub_kwargs())
        self._build_sub(self._output_dense, (query_shape[0],) + q_seq + (N, self._value_dim))

        if self.enable_ebops:
            self._beta = self.add_weight(name='beta', shape=(), initializer=self._beta0, trainable=False)
            self._ebops = self.add_weight(name='ebops', shape=(), initializer=Constant(0.0), trainable=False, dtype='uint32')
        self._q_shape = (1,) + q_seq + (N, self._key_dim)
        self._k_shape = (1,) + k_seq + (N, self._key_dim)
        self._v_shape = (1,) + k_seq + (N, self._value_dim)
        self.built = True

    def _maybe_build(self, args):
        if self.built:
            return
        q = args[0]
        self._build_device = q.device
        v = args[1] if len(args) > 1 and args[1] is not None else None
        k = args[2] if len(args) > 2 and args[2] is not None else None
        self.build(tuple(q.shape), tuple(v.shape) if v is not None else None, tuple(k.shape) if k is not None else None)

    def _ebops_loss_term(self, query_shape, value_shape=None, key_shape=None):
        # both score contractions' EBOPs from the marginal sums of the four bit-width tensors, in one launch
        if self._beta is not None and self._beta.is_cuda and self._softmax.enable_oq and self._n_seq == 1:
            (_, T, N, H), (_, S, _, Hv) = self._q_shape, self._v_shape
            operands = [self._query_dense.oq.bits_operand(self._q_shape), self._key_dense.oq.bits_operand(self._k_shape),
                        self._value_dense.oq.bits_operand(self._v_shape), self._softmax.oq.bits_operand((1, N, T, S))]
            if all(op is not None for op in operands) and N * H <= 1024 and N * S <= 2048 and sum(op[3] for op in operands) <= 30720:
                pf = float(self.parallelization_factor) if self.parallelization_factor > 0 else 1.0
                return ops.bits_ebops('mha', operands, (T, S, N, H, Hv, pf, float(self.ebops_factor)), self._beta, self._ebops)
        return super()._ebops_loss_term(query_shape, value_shape, key_shape)

    def _compute_ebops(self, query_shape, value_shape=None, key_shape=None):
        attn_shape = (1,) + tuple(self._scores_shape[1:])
        bw_q = self._query_dense.oq.bits_(self._q_shape)
        bw_k = self._key_dense.oq.bits_(self._k_shape)
        bw_v = self._value_dense.oq.bits_(self._v_shape)
        bw_attn = self._softmax.oq.bits_(attn_shape)
        ebops_qk = torch.einsum(self._dot_eq.split('->')[0] + '->', bw_k, bw_q)
        ebops_av = torch.einsum(self._combine_eq.split('->')[0] + '->', bw_attn, bw_v)
        ebops = ebops_qk + ebops_av
        if self.parallelization_factor > 0:
            return ebops * self.parallelization_factor
        return ebops

    @property
    def ebops(self):
        if self._ebops is None:
            return 0
        own = int(self._ebops.cpu().view(torch.int32))
        subs = (self._query_dense, self._key_dense, self._value_dense, self._output_dense)
        return own + sum(int(s.ebops.cpu().view(torch.int32)) for s in subs) + self._softmax.ebops

    def call(self, query, value=None, key=None, attention_mask=None, return_attention_scores=False, training=None,
             use_causal_mask=False):
        if value is None:
            value = query
        if key is None:
            key = value
        if use_causal_mask and self._n_seq != 1:
            raise NotImplementedError('use_causal_mask needs a single sequence axis')
        q = self._query_dense(query)
        k = self._key_dense(key)
        v = self._value_dense(value)
        out, scores = self._compute_attention(q, k, v, attention_mask, training, need_scores=return_attention_scores,
                                              causal=bool(use_causal_mask))
        out = self._output_dense(out)
        if self.enable_oq:
            out = self.oq(out, training=training)
        if return_attention_scores:
            return out, scores
        return out

    def _compute_attention(self, query, key, value, attention_mask=None, training=None, need_scores=True, causal=False):
        if self._inverse_sqrt_key_dim != 1.0:  # 1 after build: the scale lives in the softmax's exp table
            query = query * self._inverse_sqrt_key_dim
        flat = self._n_seq == 1
        if FUSED and flat and not need_scores and not (self._dropout and training):
            # a boolean mask [1 or B, T, S] and / or the causal rule are applied inside the kernel
            m = attention_mask
            in_kernel = m is None or (m.dim() == 3 and m.dtype == torch.bool and m.shape[0] in (1, query.shape[0])
                                      and tuple(m.shape[1:]) == (query.shape[1], key.shape[1]))
            stand_in = self._softmax.attention_plan(query, key, value, training) if in_kernel else None
            if stand_in is not None:  # one kernel each way; scores and probabilities are never written
                masks = (m, causal) if (m is not None or causal) else None
                return self._softmax(stand_in, attention=(query, key, value), attention_mask=masks), None
        if causal:
            tril = torch.tril(torch.ones((1, query.shape[1], key.shape[1]), dtype=torch.bool, device=query.device))
            attention_mask = tril if attention_mask is None else (attention_mask.bool() & tril)
        # several sequence axes, all attended: the contractions see them as one axis (same memory), the softmax and its
        # quantizers see [batch, heads, query seq..., key seq...] as the reference builds them
        B, N = query.shape[0], self._num_heads
        q_seq, k_seq = tuple(query.shape[1:-2]), tuple(key.shape[1:-2])
        q4, k4, v4 = (t.reshape(B, -1, N, t.shape[-1]) for t in (query, key, value))
        own = q4.is_cuda and max(q4.shape[1], k4.shape[1], q4.shape[3], v4.shape[3]) <= ops.ATTN_MAX
        scores = ops.attn_scores(q4, k4) if own else torch.einsum(_DOT_EQ, k4, q4)
        scores = scores.view((B, N) + q_seq + k_seq)
        mask = None
        if attention_mask is not None:
            mask = attention_mask
            while mask.dim() < scores.dim():  # broadcast over the heads (and any other axis ahead of the attended ones)
                mask = mask.unsqueeze(-2 * self._n_seq - 1)
        scores = self._softmax(scores, mask=mask)
        final = torch.nn.functional.dropout(scores, self._dropout) if (self._dropout and training) else scores
        f4 = final.reshape(B, N, q4.shape[1], k4.shape[1])
        out = ops.attn_combine(f4, v4) if own else torch.einsum(_COMBINE_EQ, f4, v4)
        return out.view((B,) + q_seq + (N, v4.shape[3])), scores
