"""CPU oracle for the HSTU block and model forward (numpy, fp64 by default).

TEST INFRASTRUCTURE ONLY: imported by tests, never by the shipped package.

Restates, in plain numpy:
  layer_norm           keras.layers.LayerNormalization as used at
                       recml/layers/keras/hstu.py:281-284 (last axis) and
                       :340-343 (axes [-2, -1]): (x - mean) / sqrt(var + eps)
                       * gamma + beta with the biased variance over the
                       normalised axes.
  hstu_block           recml/layers/keras/hstu.py:444-474 with the weights of
                       :281-354 (EinsumDense "btd,dnh->btnh" / "btnh,nhd->btd",
                       SiLU activation on U, Q, K, V, no activation on the
                       output projection).
  hstu_model           recml/layers/keras/hstu.py:585-621 (final_norm applied
                       before the blocks and again after them).
  hstu_param_count     the count asserted at recml/layers/keras/hstu_test.py:38-48.
  norm_gate            u * layer_norm(attn), hstu.py:471-472.
  gemm_silu            silu(x w + bias), the projections of hstu.py:444-449
                       (EinsumDense with activation="silu", :281-330) as one product.
  embed_norm           final_norm(scale * item_embedding[ids] + position_embedding[positions]),
                       hstu.py:593-601.
                       These three are compositions of layer_norm and hstu_oracle.silu,
                       both pinned, with a product / a row lookup.
  norm_gate_bwd        the gradients of norm_gate (and of layer_norm alone): the
                       reference leaves them to autodiff; pinned by central
                       differences of norm_gate in fp64 (tests/test_block_ops.py).

Pinning (tests/test_hstu_layer.py): layer_norm against the textbook definition
on hand-sized inputs and against torch's CPU layer_norm; the dense layers are
einsums; the attention inside is hstu_oracle.pointwise_attention_dense, pinned
in tests/test_oracle.py; hstu_param_count against the literal of the
reference's test (vocab 500, positions 20, dim 32, 3 layers -> the sum written
out there).  The reference's own tests pin only the output shape and the
parameter count of these layers, and keras / keras_hub are not importable
here, so END-TO-END PARITY of the block and model with the Keras layers is
UNPINNED: what is checked is the torch harness against this restatement.
"""

from __future__ import annotations

import numpy as np

from oracle import hstu_oracle as O


def layer_norm(x, gamma, beta, eps, axes=(-1,)):
  x = np.asarray(x, dtype=np.float64)
  mean = x.mean(axis=axes, keepdims=True)
  var = ((x - mean) ** 2).mean(axis=axes, keepdims=True)
  return (x - mean) / np.sqrt(var + eps) * np.asarray(gamma, np.float64) + np.asarray(beta, np.float64)


def hstu_block(x, w, *, num_heads, seq_lens, eps=1e-6, scaled_pointwise_attn=False,
               pos_tab=None, timestamps=None, ts_tab=None, dropout_p=0.0, dropout_seed=0):
  """x [B, L, D]; w: dict with u/q/k/v_kernel [D,H,hd], output_kernel [H,hd,D],
  input_ln_gamma/beta [D], attn_ln_gamma/beta [H,hd], optional *_bias.  dropout_p > 0: the
  block in training mode (dropout on the attention weights, hstu.py:386-387)."""
  x = np.asarray(x, dtype=np.float64)
  B, L, D = x.shape
  H = num_heads
  f = lambda name: np.asarray(w[name], dtype=np.float64)
  normed = layer_norm(x, f("input_ln_gamma"), f("input_ln_beta"), eps)
  proj = {}
  for name in ("u", "q", "k", "v"):
    y = np.einsum("btd,dnh->btnh", normed, f(f"{name}_kernel"))
    if f"{name}_bias" in w:
      y = y + f(f"{name}_bias")
    proj[name] = O.silu(y)
  mask = O.make_causal_mask((np.arange(L)[None, :] < np.asarray(seq_lens)[:, None]).astype(np.float64))
  bias = None
  if pos_tab is not None:
    bias = O.rel_pos_bias(np.asarray(pos_tab, np.float64).reshape(-1), L)
  if ts_tab is not None:
    tb = O.time_bias(np.asarray(timestamps), np.asarray(ts_tab, np.float64).reshape(-1))
    bias = tb if bias is None else bias + tb
  attn = O.pointwise_attention_dense(proj["q"], proj["k"], proj["v"], mask, bias,
                                     scaled=scaled_pointwise_attn, dropout_p=dropout_p,
                                     dropout_seed=dropout_seed)
  na = layer_norm(attn, f("attn_ln_gamma"), f("attn_ln_beta"), eps, axes=(-2, -1))
  out = np.einsum("btnh,nhd->btd", proj["u"] * na, f("output_kernel"))
  if "output_bias" in w:
    out = out + f("output_bias")
  return out + x


def hstu_model(ids, w, *, num_heads, seq_lens, eps=1e-6, scale_by_sqrt_dim=False, pos_tab=None):
  """ids [B, L]; w: item_embedding [V, D], optional position_embedding [P, D],
  final_norm_gamma/beta, blocks: list of block dicts, optional reverse_embedding [D, V]."""
  emb = np.asarray(w["item_embedding"], np.float64)[np.asarray(ids)]
  D = emb.shape[-1]
  if scale_by_sqrt_dim:
    emb = emb * D ** 0.5
  if w.get("position_embedding") is not None:
    emb = emb + np.asarray(w["position_embedding"], np.float64)[: emb.shape[1]]
  g, b = w["final_norm_gamma"], w["final_norm_beta"]
  x = layer_norm(emb, g, b, eps)
  for blk in w["blocks"]:
    x = hstu_block(x, blk, num_heads=num_heads, seq_lens=seq_lens, eps=eps, pos_tab=pos_tab)
  x = layer_norm(x, g, b, eps)
  if w.get("reverse_embedding") is None:
    return x
  return x @ np.asarray(w["reverse_embedding"], np.float64)


def hstu_param_count(vocab_size, max_positions, model_dim, num_layers, add_head=True):
  """Trainable-variable count of the reference model (hstu_test.py:38-48)."""
  d = model_dim
  n = vocab_size * d + (max_positions or 0) * d
  n += num_layers * ((d * d * 4 + d * d) + (2 * d) * 2)
  n += 2 * d
  if add_head:
    n += vocab_size * d
  return n


def norm_gate(attn, u, gamma, beta, eps=1e-6):
  """u * layer_norm(attn) over the last axis (recml/layers/keras/hstu.py:471-472)."""
  return np.asarray(u, np.float64) * layer_norm(attn, gamma, beta, eps)


def norm_gate_bwd(attn, u, gamma, beta, dout, eps=1e-6):
  """Gradients of sum(norm_gate(attn, u, gamma, beta) * dout): (d_attn, d_u, d_gamma, d_beta); u=None: of
  sum(layer_norm(attn) * dout), d_u None.  The layer norm's textbook backward: with xh the normalised row
  and g the gradient at the norm's output times gamma, d_attn = rstd (g - mean(g) - xh mean(g xh))."""
  a, do = np.asarray(attn, np.float64), np.asarray(dout, np.float64)
  gm, bt = np.asarray(gamma, np.float64), np.asarray(beta, np.float64)
  mean = a.mean(-1, keepdims=True)
  rstd = 1.0 / np.sqrt(((a - mean) ** 2).mean(-1, keepdims=True) + eps)
  xh = (a - mean) * rstd
  du = None
  gn = do
  if u is not None:
    du = do * (xh * gm + bt)
    gn = do * np.asarray(u, np.float64)
  g = gn * gm
  da = rstd * (g - g.mean(-1, keepdims=True) - xh * (g * xh).mean(-1, keepdims=True))
  red = tuple(range(a.ndim - 1))
  return da, du, (gn * xh).sum(red), gn.sum(red)


def gemm_silu(x, w, bias=None, activation=True, residual=None):
  """silu(x w + bias): the block's projections with their activation (hstu.py:444-449); without the
  activation and with `residual`, the output projection plus the block's input (hstu.py:473-474)."""
  y = np.asarray(x, np.float64) @ np.asarray(w, np.float64)
  if residual is not None:
    y = y + np.asarray(residual, np.float64)
  if bias is not None:
    y = y + np.asarray(bias, np.float64)
  return O.silu(y) if activation else y


def embed_norm(ids, table, gamma, beta, eps=1e-6, scale=1.0, positions=None, pos_table=None):
  """The model's front end (hstu.py:593-601): item row, optional scale, position row, final_norm."""
  x = np.asarray(table, np.float64)[np.asarray(ids)] * scale
  if pos_table is not None:
    x = x + np.asarray(pos_table, np.float64)[np.asarray(positions)]
  return layer_norm(x, gamma, beta, eps)
