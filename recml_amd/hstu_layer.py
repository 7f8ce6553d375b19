"""HSTU block and model forward around the MI355X attention kernel.

The harness for the end-to-end (config-4) shape: the attention is
`recml_amd.hstu_attention`, i.e. the HIP kernel behind the C ABI; in bf16
inference the projections' activation and the attention norm + U gate are the
fused steps of `recml_amd.hstu_block_ops`; the rest is plain torch on the GPU
(embedding gather, input layer norm, the output product with the residual as
its C operand).  A block built with a dropout rate drops attention weights in
training mode inside the attention kernels (forward and backward regenerate the
same keep pattern from a seed drawn per call), and the model drops embedding
entries with torch's dropout; in eval mode neither does anything.
Parameters are created frozen; after `requires_grad_(True)` the attention goes
through the HIP backward kernels; in bf16 on a GPU so do the layer norms and the
U gate (one pass each way), the attention's and the gate's gradients landing in
place in one tensor shaped like the fused projection; the matrix products and
the projections' SiLU go through torch autograd.

Mirrors, name for name:
  HSTUBlock   recml/layers/keras/hstu.py:240-474 (weights :281-354, call :422-474)
  HSTU        recml/layers/keras/hstu.py:492-621 (call :585-621)

Differences from the reference layer, on purpose:
  * the [B, L, L] attention mask and bias tensors are never built: the block
    takes `seq_lens` (end-padded batches, as the reference's data pipeline
    produces) and the bias *tables* (`pos_bias`, `timestamps` + `ts_bias`);
  * U, Q, K, V come from one fused [D, 4D] GEMM; the four kernels are stored
    separately under the reference's names and concatenated at call time;
  * softmax attention (hstu.py:392-420) is not implemented here.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from recml_amd import hstu_block_ops
from recml_amd import hstu_ops
from recml_amd import masks


def _wants_grad(*tensors) -> bool:
  return torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors)


def _attention(q, k, v, *, pos_bias=None, ts_bias=None, batch=None, **kw):
  """The attention op, differentiable when anything it reads wants a gradient: through the HIP
  backward kernels for q, k, v, the bias tables and a dense bias.  `batch`: the per-batch preparation
  shared by the layers (inference only)."""
  if _wants_grad(q, k, v, pos_bias, ts_bias, kw.get("bias")):
    return hstu_ops.hstu_attention_autograd(q, k, v, pos_bias=pos_bias, ts_bias=ts_bias, **kw)
  return hstu_ops.hstu_attention(q, k, v, pos_bias=pos_bias, ts_bias=ts_bias, batch=batch, **kw)


class _AttentionGateFn(torch.autograd.Function):
  """gated = u * layer_norm(attention(q, k, v)) on the four slices of ONE fused projection
  uqkv [..., 4, H, hd] (contiguous, bf16), with every gradient through the HIP kernels.

  One function instead of a chain of three because of what the chain costs on the way back: the
  gradients of the four slices come back as four tensors that autograd then copies into one (a pass
  over 4 x tokens x D per block).  Here the backward kernels write them where they belong: the
  attention's dq, dk, dv and the gate's du straight into the slices of one gradient tensor shaped
  like the projection."""

  @staticmethod
  def forward(ctx, uqkv, gamma, beta, pos_bias, ts_bias, eps, batch, kwargs):
    uqkv = uqkv.contiguous()            # (the backward mirrors this layout for the gradient)
    u, q, k, v = uqkv.unbind(dim=-3)
    attn = hstu_ops.hstu_attention(q, k, v, pos_bias=pos_bias, ts_bias=ts_bias, batch=batch, **kwargs)
    W = q.shape[-2] * q.shape[-1]
    gated = hstu_block_ops.norm_gate(attn.reshape(-1, W).detach(), u.reshape(-1, W).detach(), gamma.detach().reshape(-1),
                                     beta.detach().reshape(-1), eps)
    ctx.save_for_backward(uqkv, attn, gamma, beta, *(t for t in (pos_bias, ts_bias) if t is not None))
    ctx.has = (pos_bias is not None, ts_bias is not None)
    ctx.eps, ctx.kwargs = eps, kwargs
    return gated.reshape(*uqkv.shape[:-3], W)

  @staticmethod
  def backward(ctx, dgated):
    uqkv, attn, gamma, beta, *rest = ctx.saved_tensors
    pos = rest.pop(0) if ctx.has[0] else None
    ts = rest.pop(0) if ctx.has[1] else None
    u, q, k, v = uqkv.unbind(dim=-3)
    W = q.shape[-2] * q.shape[-1]
    d_uqkv = torch.empty_like(uqkv)                     # uqkv is contiguous: the same strides
    du, dq, dk, dv = d_uqkv.unbind(dim=-3)
    du2 = du.reshape(-1, W)
    assert du2.data_ptr() == du.data_ptr()              # a view: the kernel writes into d_uqkv
    d_attn, _, dg, db = hstu_block_ops.norm_gate_bwd(attn.reshape(-1, W), u.reshape(-1, W), gamma.reshape(-1), beta.reshape(-1),
                                                     dgated.reshape(-1, W).contiguous(), ctx.eps, du_out=du2)
    # needs_input_grad follows forward's arguments: uqkv, gamma, beta, pos_bias, ts_bias, ...
    want_tables = (pos is not None and ctx.needs_input_grad[3]) or (ts is not None and ctx.needs_input_grad[4])
    _, _, _, dpos, dts = hstu_ops.hstu_attention_bwd(q, k, v, d_attn.reshape(attn.shape), pos_bias=pos, ts_bias=ts,
                                                     table_grads=want_tables, grads_out=(dq, dk, dv), **ctx.kwargs)
    cast = lambda g, t: None if g is None else g.to(t.dtype)
    return (d_uqkv, dg.to(gamma.dtype).reshape(gamma.shape), db.to(beta.dtype).reshape(beta.shape),
            cast(dpos, pos) if pos is not None else None, cast(dts, ts) if ts is not None else None, None, None, None)


class _OutputProjectionFn(torch.autograd.Function):
  """gated @ W (+ bias) + residual with the residual as the product's C operand (recml/layers/keras/hstu.py:473-474):
  torch's addmm copies the residual into the output before the product.  The gradients are two plain products."""

  @staticmethod
  def forward(ctx, gated, w, bias, residual):
    ctx.save_for_backward(gated, w)
    ctx.has_bias = bias is not None
    return hstu_block_ops.gemm_silu(gated, w, bias, False, residual=residual)

  @staticmethod
  def backward(ctx, dout):
    gated, w = ctx.saved_tensors
    need = ctx.needs_input_grad
    d_gated = dout @ w.t() if need[0] else None
    d_w = gated.t() @ dout if need[1] else None
    d_bias = dout.sum(0) if (ctx.has_bias and need[2]) else None
    return d_gated, d_w, d_bias, dout if need[3] else None


def _glorot_uniform(shape, fan_in, fan_out, generator, dtype, device):
  limit = math.sqrt(6.0 / (fan_in + fan_out))
  w = torch.empty(shape, dtype=torch.float32)
  w.uniform_(-limit, limit, generator=generator)
  return w.to(device=device, dtype=dtype)


class HSTUBlock(torch.nn.Module):
  """One HSTU block: LN -> U,Q,K,V = act(x W) -> pointwise attention -> LN over
  (heads, head_dim) -> U * normed -> output projection -> + inputs
  (recml/layers/keras/hstu.py:444-474)."""

  def __init__(self, hidden_dim: int, num_heads: int, use_bias: bool = False,
               layer_norm_epsilon: float = 1e-6, scaled_pointwise_attn: bool = False,
               softmax_attention: bool = False, dropout: float = 0.0,
               dtype=torch.float32, device=None, generator=None):
    super().__init__()
    if softmax_attention:
      raise NotImplementedError("softmax attention is outside this build; only the pointwise path is accelerated")
    if hidden_dim % num_heads:
      raise ValueError(f"hidden_dim {hidden_dim} is not a multiple of num_heads {num_heads}")
    if not 0.0 <= dropout < 1.0:
      raise ValueError(f"dropout must be in [0, 1), got {dropout}")
    # The reference drops attention weights in training (recml/layers/keras/hstu.py:386-387): here the attention
    # kernels do it, from a seed this block draws per forward.
    self.dropout = float(dropout)
    self.num_heads = num_heads
    self.head_dim = hidden_dim // num_heads
    self.hidden_dim = hidden_dim
    self.eps = layer_norm_epsilon
    self.scaled_pointwise_attn = scaled_pointwise_attn
    H, hd, D = num_heads, self.head_dim, hidden_dim
    P = torch.nn.Parameter
    # EinsumDense "btd,dnh->btnh": kernel [D, H, hd], Glorot-uniform with the fans Keras
    # computes for a rank-3 shape (see _fans)
    fi, fo = self._fans((D, H, hd))
    for name in ("u", "q", "k", "v"):
      self.register_parameter(f"{name}_kernel", P(_glorot_uniform((D, H, hd), fi, fo, generator, dtype, device), requires_grad=False))
      if use_bias:
        self.register_parameter(f"{name}_bias", P(torch.zeros((H, hd), dtype=dtype, device=device), requires_grad=False))
    fi, fo = self._fans((H, hd, D))
    self.output_kernel = P(_glorot_uniform((H, hd, D), fi, fo, generator, dtype, device), requires_grad=False)
    self.output_bias = P(torch.zeros((D,), dtype=dtype, device=device), requires_grad=False) if use_bias else None
    self.use_bias = use_bias
    self.input_ln_gamma = P(torch.ones((D,), dtype=dtype, device=device), requires_grad=False)
    self.input_ln_beta = P(torch.zeros((D,), dtype=dtype, device=device), requires_grad=False)
    self.attn_ln_gamma = P(torch.ones((H, hd), dtype=dtype, device=device), requires_grad=False)
    self.attn_ln_beta = P(torch.zeros((H, hd), dtype=dtype, device=device), requires_grad=False)

  @staticmethod
  def _fans(shape):
    """Keras' fan computation for a rank-3 kernel: the leading axes are the
    receptive field (keras/src/initializers/random_initializers.py,
    compute_fans): fan_in = shape[-2] * prod(shape[:-2]), fan_out = shape[-1] * prod(shape[:-2])."""
    rf = 1
    for s in shape[:-2]:
      rf *= s
    return shape[-2] * rf, shape[-1] * rf

  def _dropout_kw(self, dropout_seed=None) -> dict:
    """The attention's dropout arguments for this call: none in eval mode or at rate 0; in training mode the
    block's rate and a seed from torch's CPU generator (so torch.manual_seed makes a run repeatable, and no GPU
    work waits on it) unless the caller brings one."""
    if not (self.training and self.dropout > 0.0):
      return {}
    if dropout_seed is None:
      dropout_seed = int(torch.randint(0, 2 ** 62, (1,)).item())
    return dict(dropout_p=self.dropout, dropout_seed=int(dropout_seed))

  def forward(self, inputs, *, seq_lens=None, pos_bias=None, timestamps=None, ts_bias=None,
              attention_mask=None, attention_bias=None, batch=None, dropout_seed=None):
    """inputs [B, L, D] -> [B, L, D].

    Give `seq_lens` [B] (keys and rows at or past the length are masked, as
    make_causal_mask does for an end-padded batch) with optional bias tables;
    or, for the reference's calling convention, a dense `attention_mask`
    [B, L, L] and optional `attention_bias` [B, L, L]
    (recml/layers/keras/hstu.py:422-440).  `batch`: an `hstu_ops.AttentionBatch` shared with the
    other blocks that see the same lengths, timestamps and tables.  `dropout_seed`: in training mode
    with a dropout rate, the seed of this call's keep pattern (default: drawn from torch's generator).
    """
    drop = self._dropout_kw(dropout_seed)
    B, L, D = inputs.shape
    H, hd = self.num_heads, self.head_dim
    fused = self._fused_inference(inputs, pos_bias, ts_bias, attention_bias)
    if attention_mask is None and attention_bias is None and self._fused_training(inputs, pos_bias, ts_bias):
      alpha, n = (1.0 / math.sqrt(hd), 1.0) if self.scaled_pointwise_attn else (1.0, float(L))
      return self._train_steps(inputs.reshape(B * L, D), (B, L), pos_bias, ts_bias, batch,
                               dict(seq_lens=seq_lens, n=n, alpha=alpha, timestamps=timestamps, **drop)).reshape(B, L, D)
    x = self._input_norm(inputs, fused)
    w, b = self._uqkv_weights()
    if fused:
      uqkv = hstu_block_ops.gemm_silu(x.reshape(B * L, D), w, b, True).reshape(B, L, 4, H, hd)
    else:
      uqkv = x.reshape(B * L, D) @ w
      if b is not None:
        uqkv = uqkv + b
      uqkv = F.silu(uqkv).reshape(B, L, 4, H, hd)
    u, q, k, v = uqkv.unbind(dim=2)
    if attention_mask is not None:
      # the reference's calling convention: a dense [B, L, L] mask and bias (training: forward and backward kernels,
      # the gradient of a dense bias included)
      attn = hstu_ops.pointwise_attention(q, k, v, attention_mask, attention_bias,
                                          scaled_pointwise_attn=self.scaled_pointwise_attn, batch=batch, **drop)
    else:
      alpha, n = (1.0 / math.sqrt(hd), 1.0) if self.scaled_pointwise_attn else (1.0, float(L))
      attn = _attention(q, k, v, seq_lens=seq_lens, n=n, alpha=alpha, pos_bias=pos_bias,
                        timestamps=timestamps, ts_bias=ts_bias, bias=attention_bias, batch=batch, **drop)
    if fused:
      gated = hstu_block_ops.norm_gate(attn.reshape(B * L, H * hd), u.reshape(B * L, H * hd), self.attn_ln_gamma.reshape(-1),
                                       self.attn_ln_beta.reshape(-1), self.eps)
      return hstu_block_ops.gemm_silu(gated, self.output_kernel.reshape(H * hd, D), self.output_bias, False,
                                      residual=inputs.reshape(B * L, D)).reshape(B, L, D)
    normed = F.layer_norm(attn.reshape(B, L, H * hd), (H * hd,), self.attn_ln_gamma.reshape(-1),
                          self.attn_ln_beta.reshape(-1), self.eps)
    gated = u.reshape(B, L, H * hd) * normed
    out = gated.reshape(B * L, H * hd) @ self.output_kernel.reshape(H * hd, D)
    if self.use_bias:
      out = out + self.output_bias
    return out.reshape(B, L, D) + inputs


  def _fused_inference(self, t, *bias_inputs) -> bool:
    """Whether the fused block steps apply: bf16 on a GPU, nothing asking for gradients (the fused
    steps are not differentiable: a bias table or dense bias that requires a gradient rules them out
    like a parameter of the block would)."""
    wants_grad = _wants_grad(t, *self.parameters(), *bias_inputs)
    return t.is_cuda and t.dtype == torch.bfloat16 and not wants_grad

  def _input_norm(self, t, fused):
    D = self.hidden_dim
    if fused and D % 8 == 0 and D <= 8192:
      return hstu_block_ops.layer_norm(t, self.input_ln_gamma, self.input_ln_beta, self.eps)   # one wave per row, one pass
    return F.layer_norm(t, (D,), self.input_ln_gamma, self.input_ln_beta, self.eps)

  def _fused_training(self, t, *bias_inputs) -> bool:
    """Whether the training form of the fused steps applies: bf16 on a GPU, something asking for a
    gradient, widths the norm kernels' backward takes."""
    D, W = self.hidden_dim, self.num_heads * self.head_dim
    return (t.is_cuda and t.dtype == torch.bfloat16 and _wants_grad(t, *self.parameters(), *bias_inputs)
            and D % 8 == 0 and W % 8 == 0 and D <= 2048 and W <= 2048)

  def _train_steps(self, tokens, lead, pos_bias, ts_bias, batch, attn_kw):
    """The block on rows [T, D] with gradients: input norm, attention + attention norm + U gate (one
    function whose backward writes the projection's gradient in place) through the HIP kernels forward
    and backward; the two matrix products and the projections' SiLU through torch.  `lead`: the leading
    shape of the attention's tensors ((B, L) padded, (T,) packed)."""
    H, hd = self.num_heads, self.head_dim
    x = hstu_block_ops.layer_norm(tokens, self.input_ln_gamma, self.input_ln_beta, self.eps)
    w, b = self._uqkv_weights()
    uqkv = x @ w
    if b is not None:
      uqkv = uqkv + b
    uqkv = F.silu(uqkv).reshape(*lead, 4, H, hd)
    gated = _AttentionGateFn.apply(uqkv, self.attn_ln_gamma, self.attn_ln_beta, pos_bias, ts_bias, self.eps, batch, attn_kw)
    return _OutputProjectionFn.apply(gated.reshape(-1, H * hd), self.output_kernel.reshape(H * hd, self.hidden_dim),
                                     self.output_bias, tokens)

  def _uqkv_weights(self):
    w = torch.cat([self.u_kernel, self.q_kernel, self.k_kernel, self.v_kernel], dim=1).reshape(self.hidden_dim, -1)
    b = torch.cat([self.u_bias, self.q_bias, self.k_bias, self.v_bias], dim=0).reshape(-1) if self.use_bias else None
    return w, b

  def forward_jagged(self, tokens, seq_offsets, max_len, *, pos_bias=None, timestamps=None, ts_bias=None, batch=None,
                     dropout_seed=None):
    """The block on packed tokens [T, D] (sequence b = rows seq_offsets[b]..seq_offsets[b+1]):
    no work at all for padding, in the projections either.  `timestamps` is jagged [T].

    Inference in bf16 takes the fused steps: the projections' SiLU in the epilogue of their one
    matrix product, the attention norm and the U gate in one pass (recml_amd.hstu_block_ops), the
    residual as the C operand of the output product."""
    drop = self._dropout_kw(dropout_seed)
    T, D = tokens.shape
    H, hd = self.num_heads, self.head_dim
    fused = self._fused_inference(tokens, pos_bias, ts_bias)
    if self._fused_training(tokens, pos_bias, ts_bias):
      alpha, n = (1.0 / math.sqrt(hd), 1.0) if self.scaled_pointwise_attn else (1.0, float(max_len))
      return self._train_steps(tokens, (T,), pos_bias, ts_bias, batch,
                               dict(seq_offsets=seq_offsets, max_len=max_len, n=n, alpha=alpha, timestamps=timestamps, **drop))
    x = self._input_norm(tokens, fused)
    w, b = self._uqkv_weights()
    if fused:
      uqkv = hstu_block_ops.gemm_silu(x, w, b, True).reshape(T, 4, H, hd)
    else:
      uqkv = x @ w
      if b is not None:
        uqkv = uqkv + b
      uqkv = F.silu(uqkv).reshape(T, 4, H, hd)
    u, q, k, v = uqkv.unbind(dim=1)
    alpha, n = (1.0 / math.sqrt(hd), 1.0) if self.scaled_pointwise_attn else (1.0, float(max_len))
    attn = _attention(q, k, v, seq_offsets=seq_offsets, max_len=max_len, n=n, alpha=alpha,
                      pos_bias=pos_bias, timestamps=timestamps, ts_bias=ts_bias, batch=batch, **drop)
    if fused:
      gated = hstu_block_ops.norm_gate(attn.reshape(T, H * hd), u.reshape(T, H * hd), self.attn_ln_gamma.reshape(-1),
                                       self.attn_ln_beta.reshape(-1), self.eps)
      return hstu_block_ops.gemm_silu(gated, self.output_kernel.reshape(H * hd, D), self.output_bias, False, residual=tokens)
    normed = F.layer_norm(attn.reshape(T, H * hd), (H * hd,), self.attn_ln_gamma.reshape(-1),
                          self.attn_ln_beta.reshape(-1), self.eps)
    out = (u.reshape(T, H * hd) * normed) @ self.output_kernel.reshape(H * hd, D)
    if self.use_bias:
      out = out + self.output_bias
    return out + tokens


class HSTU(torch.nn.Module):
  """The HSTU model forward (recml/layers/keras/hstu.py:585-621): item
  embedding (x sqrt(D)) + position embedding -> final_norm -> blocks ->
  final_norm (the same layer both times) -> optional untied output head."""

  def __init__(self, *, vocab_size: int, max_positions: int | None = None, model_dim: int,
               num_heads: int, num_layers: int, dropout: float = 0.0, norm_eps: float = 1e-6,
               scale_by_sqrt_dim: bool = False, add_head: bool = True,
               dtype=torch.float32, device=None, seed: int = 0):
    super().__init__()
    g = torch.Generator().manual_seed(seed)
    P = torch.nn.Parameter
    normal = lambda shape: (torch.randn(shape, generator=g) * 0.02).to(device=device, dtype=dtype)
    self.item_embedding = P(normal((vocab_size, model_dim)), requires_grad=False)
    self.position_embedding = P(normal((max_positions, model_dim)), requires_grad=False) if max_positions else None
    self.decoder_blocks = torch.nn.ModuleList(
        HSTUBlock(model_dim, num_heads, layer_norm_epsilon=norm_eps, dropout=dropout, dtype=dtype, device=device, generator=g)
        for _ in range(num_layers))
    self.final_norm_gamma = P(torch.ones((model_dim,), dtype=dtype, device=device), requires_grad=False)
    self.final_norm_beta = P(torch.zeros((model_dim,), dtype=dtype, device=device), requires_grad=False)
    self.reverse_embedding = P(normal((model_dim, vocab_size)), requires_grad=False) if add_head else None
    self.model_dim = model_dim
    self.eps = norm_eps
    self.scale_by_sqrt_dim = scale_by_sqrt_dim
    self.dropout = float(dropout)      # on the embeddings here (hstu.py:541-543, 602), on the attention weights in the blocks

  def count_params(self) -> int:
    return sum(p.numel() for p in self.parameters())

  def _final_norm(self, x):
    D = self.model_dim
    training = _wants_grad(x, self.final_norm_gamma, self.final_norm_beta)
    if x.is_cuda and x.dtype == torch.bfloat16 and D % 8 == 0 and D <= (2048 if training else 8192):
      # bf16 on a GPU: the norm (and its gradients) in one pass each
      return hstu_block_ops.layer_norm(x, self.final_norm_gamma, self.final_norm_beta, self.eps)
    return F.layer_norm(x, (D,), self.final_norm_gamma, self.final_norm_beta, self.eps)

  def _fused_front_end(self) -> bool:
    """bf16 inference on a GPU: gather, scale, position embedding and final_norm as one pass."""
    t = self.item_embedding
    wants_grad = torch.is_grad_enabled() and any(
        p is not None and p.requires_grad
        for p in (self.item_embedding, self.position_embedding, self.final_norm_gamma, self.final_norm_beta))
    return t.is_cuda and t.dtype == torch.bfloat16 and not wants_grad

  def _embed_norm(self, ids, positions):
    scale = self.model_dim ** 0.5 if self.scale_by_sqrt_dim else 1.0
    return hstu_block_ops.embed_norm(ids.to(torch.int64), self.item_embedding, self.final_norm_gamma, self.final_norm_beta,
                                     self.eps, scale=scale, positions=None if positions is None else positions.to(torch.int64),
                                     pos_table=self.position_embedding)

  def forward(self, inputs, padding_mask=None, attention_mask=None, *, seq_lens=None, pos_bias=None, timestamps=None,
              ts_bias=None, jagged=False):
    """inputs: item ids [B, L]; `padding_mask` [B, L] (1 = real item, end-padded) or `seq_lens` [B]; or, as
    the reference's call also allows (hstu.py:585-615), a dense `attention_mask` [B, L, L] that every block
    then takes as it is (any mask, at the price of reading it in every layer).

    jagged=True packs the valid tokens once and runs every block on [T, D]: nothing is computed
    for padding.  Rows past a sequence's length are then returned as zeros, whereas the padded
    form (like the reference) carries the padded positions' own embeddings through the blocks.
    """
    if attention_mask is not None:
      if jagged or pos_bias is not None or ts_bias is not None or seq_lens is not None:
        raise ValueError("`attention_mask` goes with the padded form and without `seq_lens` and bias tables")
    elif seq_lens is None:
      if padding_mask is None:
        raise ValueError("Either `attention_mask`, `padding_mask` or `seq_lens` must be set.")
      seq_lens = masks.lengths_from_padding_mask(padding_mask)
    if jagged:
      return self._forward_jagged(inputs, seq_lens, pos_bias, timestamps, ts_bias)
    if self._fused_front_end():
      pos = None
      if self.position_embedding is not None:
        pos = torch.arange(inputs.shape[1], device=inputs.device)[None, :].expand(inputs.shape).contiguous()
      x = self._embed_norm(inputs, pos)
    else:
      x = self.item_embedding[inputs]
      if self.scale_by_sqrt_dim:
        x = x * (self.model_dim ** 0.5)
      if self.position_embedding is not None:
        x = x + self.position_embedding[: x.shape[1]]
      x = self._final_norm(x)
    x = F.dropout(x, self.dropout, self.training)
    # every block sees the same lengths, timestamps and tables: the attention prepares them once
    batch = hstu_ops.AttentionBatch()
    for block in self.decoder_blocks:
      if attention_mask is not None:
        x = block(x, attention_mask=attention_mask, batch=batch)
      else:
        x = block(x, seq_lens=seq_lens, pos_bias=pos_bias, timestamps=timestamps, ts_bias=ts_bias, batch=batch)
    x = self._final_norm(x)
    if self.reverse_embedding is None:
      return x
    return x @ self.reverse_embedding

  def _forward_jagged(self, inputs, seq_lens, pos_bias, timestamps, ts_bias):
    B, L = inputs.shape
    lens = seq_lens.to(torch.int64).clamp(0, L)
    valid = torch.arange(L, device=inputs.device)[None, :] < lens[:, None]          # [B, L]
    offsets = torch.zeros(B + 1, dtype=torch.int32, device=inputs.device)
    offsets[1:] = torch.cumsum(lens, 0)
    # the flat positions of the valid tokens, sequence-major: found once (the one host wait of the packing:
    # the token count) and used for every gather and for the scatter at the end
    where = valid.reshape(-1).nonzero().squeeze(1)                                   # [T]
    ids = inputs.reshape(-1)[where]
    pos_idx = where % L if self.position_embedding is not None else None
    if self._fused_front_end():
      x = self._embed_norm(ids, pos_idx)
    else:
      x = self.item_embedding[ids]
      if self.scale_by_sqrt_dim:
        x = x * (self.model_dim ** 0.5)
      if pos_idx is not None:
        x = x + self.position_embedding[pos_idx]
      x = self._final_norm(x)
    x = F.dropout(x, self.dropout, self.training)
    ts = None if timestamps is None else timestamps.reshape(-1)[where]
    batch = hstu_ops.AttentionBatch()
    for block in self.decoder_blocks:
      x = block.forward_jagged(x, offsets, L, pos_bias=pos_bias, timestamps=ts, ts_bias=ts_bias, batch=batch)
    x = self._final_norm(x)
    if self.reverse_embedding is not None:
      x = x @ self.reverse_embedding
    out = torch.zeros((B * L, x.shape[-1]), dtype=x.dtype, device=x.device)
    return out.index_copy(0, where, x).reshape(B, L, x.shape[-1])
