"""Layers: compositions of Tensor ops, parameter shapes and initial distributions as in
dlgrad/nn/__init__.py:8-41."""
import math

from dlgrad_amd import ops
from dlgrad_amd.buffer import Buffer
from dlgrad_amd.device import Device
from dlgrad_amd.nn import optim, utils  # noqa: F401
from dlgrad_amd.tensor import Tensor
from dlgrad_amd.nn import datasets  # noqa: E402,F401  (uses Tensor)


class Linear:
    """y = x @ W^T + b with W (out, in) and b (1, out), both U(-1/sqrt(in), 1/sqrt(in))."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device: Device = Device.CPU) -> None:
        bound = 1 / math.sqrt(in_features)
        self.weight = Tensor.uniform((out_features, in_features), low=-bound, high=bound,
                                     requires_grad=True, device=device)
        self.bias = Tensor.uniform((1, out_features), low=-bound, high=bound,
                                   requires_grad=True, device=device) if bias else None

    def __call__(self, x: Tensor, residual: Tensor | None = None) -> Tensor:
        """x @ W^T + b, plus `residual` if given (an extension: on the hip device the addition is
        part of the product kernel, ops.LinearNTAdd)."""
        if residual is None:
            return x.linear(self.weight, self.bias)
        if self.bias is None and residual.shape == x.shape[:-1] + (self.weight.shape[0],) \
                and residual.device is x.device and ops.use_fused_epilogues(x, self.weight):
            return ops.LinearNTAdd.execute(x, self.weight, residual)
        return residual + x.linear(self.weight, self.bias)


class Embedding:
    """Row lookup in a (num_embeddings, embedding_dim) table initialised U[0, 1); indices
    are fp32-encoded integers."""

    def __init__(self, num_embeddings: int, embedding_dim: int, device: Device = Device.CPU) -> None:
        self.num_embeddings, self.embedding_dim = num_embeddings, embedding_dim
        self.weight = Tensor.uniform((num_embeddings, embedding_dim), requires_grad=True, device=device)

    def __call__(self, idx: Tensor) -> Tensor:
        return Tensor.embedding(self.weight, idx)


class RMSNorm:
    """x * rsqrt(mean(x^2, last, keepdim) + eps) * weight, weight (1, dim) of ones."""

    def __init__(self, dim: int, eps: float = 1e-6, elementwise_affine: bool = True,
                 device: Device = Device.CPU) -> None:
        self.eps = eps
        self.weight = Tensor.ones((1, dim), device=device, requires_grad=True) if elementwise_affine else None

    def _norm(self, x: Tensor) -> Tensor:
        ms = (x ** 2).mean(x.ndim - 1, keepdim=True)
        return x * (ms + self.eps).rsqrt()

    def __call__(self, x: Tensor) -> Tensor:
        if ops.use_fused_rmsnorm(x, self.weight):
            args = (x,) if self.weight is None else (x, self.weight)
            return ops.RMSNorm.execute(*args, eps=self.eps)
        y = self._norm(x)
        return y if self.weight is None else y * self.weight


def causal_attention(q: Tensor, k: Tensor, v: Tensor, scale: float) -> Tensor:
    """softmax(causal_mask(q @ k^T * scale)) @ v over the last two dims of q, k (.., T, d) and
    v (.., T, dv): the no-cache branch of the reference's attention (examples/gpt.py:50-55).
    On the hip device it is one graph node that runs the chain's kernels with the causal
    structure known (ops.CausalAttention: same values, about half the work); elsewhere it is
    the chain itself."""
    if ops.use_fused_causal_attention(q, k, v):
        return ops.CausalAttention.execute(q, k, v, scale=scale)
    nd, T = q.ndim, q.shape[-2]
    mask = Tensor(ops.causal_mask(T, q.device))
    return (q @ k.transpose(nd - 2, nd - 1)).masked_softmax(mask, scale, dim=nd - 1) @ v


def causal_self_attention(q: Tensor, k: Tensor, v: Tensor, n_head: int, scale: float) -> Tensor:
    """Multi-head causal attention on the projections themselves: q, k, v and the result are
    (B, T, n_head * d).  What examples/gpt.py:45-57 writes as reshape -> transpose(1, 2) for each of
    q, k, v, the attention, and transpose(1, 2) -> reshape back.  On the hip device the heads
    are read and written in place (ops.CausalAttentionHeads); elsewhere it is that sequence."""
    if ops.use_fused_attention_heads(q, k, v, n_head):
        return ops.CausalAttentionHeads.execute(q, k, v, n_head=n_head, scale=scale)
    B, T, C = q.shape
    split = (B, T, n_head, C // n_head)
    qh, kh, vh = (t.reshape(split).transpose(1, 2) for t in (q, k, v))
    return causal_attention(qh, kh, vh, scale).transpose(1, 2).reshape((B, T, C))


def cached_attention(q: Tensor, k_store: Tensor, v_store: Tensor, n: int, n_head: int, scale: float,
                     hidden: Tensor | None = None) -> Tensor:
    """Attention of one new position per sequence over a key/value cache, for inference: q is the
    (B, 1, C) query projection, k_store and v_store are (block, B, C) with the first n rows in use,
    `hidden` (1, 1, 1, n) marks rows to leave out.  The else-branch of the reference's attention
    (examples/gpt.py:58-63) without its host concatenation.  On the hip device the heads are read
    in place from q and from the stores; elsewhere the views are materialised as there."""
    B, _, C = q.shape
    if ops.FUSED and q.device is Device.HIP and k_store.device is Device.HIP and v_store.device is Device.HIP \
            and ops.softmax_row_fits(n):
        h = None if hidden is None else hidden.data
        return Tensor(q.data.cached_attention(k_store.data, v_store.data, n, n_head, scale, h))
    split = (n, B, n_head, C // n_head)
    k = k_store[0:n].reshape(split).permute((1, 2, 0, 3))                  # (B, h, n, d)
    v = v_store[0:n].reshape(split).permute((1, 2, 0, 3))
    qh = q.reshape((B, 1, n_head, C // n_head)).transpose(1, 2)            # (B, h, 1, d)
    att = qh @ k.transpose(2, 3)
    att = (att * scale).softmax(dim=3) if hidden is None else att.masked_softmax(hidden, scale, dim=3)
    return (att @ v).transpose(1, 2).reshape((B, 1, C))


def stack_parameters(tensors: list) -> None:
    """Moves the data of equally shaped parameter tensors into one allocation, back to back in the
    given order (values kept, each tensor now a view of its part).  Nothing else about them
    changes -- names, shapes, gradients, optimizer and checkpoint handling -- but kernels may
    treat them as one matrix: see self_attention_qkv.  A no-op off the hip device."""
    first = tensors[0]
    if first.device is not Device.HIP or any(t.shape != first.shape or t.device is not Device.HIP for t in tensors):
        return
    n = first.numel
    base = Buffer.full((len(tensors) * n,), 0.0, Device.HIP)
    for i, t in enumerate(tensors):
        part = Buffer(base.ptr + i * n, t.shape, Device.HIP)
        part.copy_(t.data)
        t.data = part


def self_attention_qkv(x: Tensor, wq: Tensor, wk: Tensor, wv: Tensor, n_head: int, scale: float, norm=None) -> Tensor:
    """causal_self_attention(x @ wq^T, x @ wk^T, x @ wv^T, n_head, scale) for x (B, T, C) and three
    (C, C) weights: the projections and attention of examples/gpt.py:45-57.  When the weights are
    stacked in memory (stack_parameters) the hip device runs one projection and reads q, k, v out
    of its result in place (ops.SelfAttentionQKV).  norm: an RMSNorm to apply to x first; where the
    one-projection form runs and the rows are short enough, that projection applies it."""
    if ops.use_fused_qkv_attention(x, wq, wk, wv, n_head):
        if norm is not None and ops.tile_norm_applies(x, wq, norm):
            return ops.SelfAttentionQKV.execute(x, wq, wk, wv, norm.weight, n_head=n_head, scale=scale, eps=norm.eps)
        return ops.SelfAttentionQKV.execute(x if norm is None else norm(x), wq, wk, wv, n_head=n_head, scale=scale)
    if norm is not None:
        x = norm(x)
    return causal_self_attention(x.linear(wq, None), x.linear(wk, None), x.linear(wv, None), n_head, scale)


_inference_depth = 0


class inference:
    """with nn.inference(): ... -- the caller states that nothing computed inside will be differentiated.
    The single-row decoding forms of norm_linear, mlp_relu and project_qkv_row return results without a
    tape; outside such a block they are taken only when no input asks for a gradient, so that a training
    forward over a single row (a (1, 1) batch) keeps its graph."""

    def __enter__(self):
        global _inference_depth
        _inference_depth += 1
        return self

    def __exit__(self, *exc):
        global _inference_depth
        _inference_depth -= 1
        return False


def _tape_free(*tensors) -> bool:
    """May a result of these inputs go without a tape?  Inside nn.inference(), or when none of them requires a gradient."""
    return _inference_depth > 0 or not any(t is not None and t.requires_grad for t in tensors)


def _row_norm(x: Tensor, w: Buffer, norm) -> tuple | None:
    """(gain, eps) if the product of the single row x with w^T can RMS-normalise x on the way (hip device,
    a norm with a gain, a row that fits the kernel), else None: the caller then applies the norm itself."""
    if norm is None or norm.weight is None or not ops.FUSED or x.device is not Device.HIP or norm.weight.device is not Device.HIP:
        return None
    from dlgrad_amd.runtime.hip import HIP
    return (norm.weight.data, norm.eps) if HIP.row_norm_fits(x.data, w, norm.weight.data) else None


def project_qkv_row(x: Tensor, wq: Tensor, wk: Tensor, wv: Tensor, norm=None) -> tuple[Tensor, Tensor, Tensor]:
    """(x @ wq^T, x @ wk^T, x @ wv^T) for decoding.  When x is a single row and the weights are stacked
    in memory (stack_parameters), the hip device runs one product and the three results are the
    thirds of its output row; such results carry no tape (inference only).  Otherwise three linears.
    norm: an RMSNorm to apply to x first; in the one-product case it is applied inside the product."""
    if x.numel == x.shape[-1] and x.numel and ops.FUSED and ops.stacked(wq, wk, wv) and x.device is wq.device \
            and _tape_free(x, wq, wk, wv, None if norm is None else norm.weight):
        C = wq.shape[0]
        w = Buffer(wq.data.ptr, (3 * C, wq.shape[1]), wq.device)
        inside = _row_norm(x, w, norm)
        row = x.data.matmul_nt(w, norm=inside) if inside else (x if norm is None else norm(x)).data.matmul_nt(w)
        shape = x.shape[:-1] + (C,)
        return tuple(Tensor(Buffer(row.ptr + i * C, shape, x.device), requires_grad=False) for i in range(3))
    if norm is not None:
        x = norm(x)
    return x.linear(wq, None), x.linear(wk, None), x.linear(wv, None)


def embed_tokens(wte: "Embedding", wpe: "Embedding", idx: Tensor, pos: Tensor) -> Tensor:
    """wte(idx) + wpe(pos) for token ids idx (B, T) and position ids pos (T,): the first line of a transformer's
    forward (examples/gpt.py:96-98).  On the hip device one node and one launch, bit-identical to the three ops;
    elsewhere the three ops."""
    if ops.FUSED and idx.ndim == 2 and pos.ndim == 1 and pos.numel == idx.shape[1] and wte.weight.ndim == 2 \
            and wpe.weight.ndim == 2 and wte.weight.shape[1] == wpe.weight.shape[1] \
            and all(t.device is Device.HIP for t in (wte.weight, wpe.weight, idx, pos)):
        return ops.EmbeddingSum.execute(wte.weight, wpe.weight, idx, pos)
    return wte(idx) + wpe(pos)


def _decode_fused(*tensors: Tensor) -> bool:
    if not ops.FUSED or any(t.device is not Device.HIP for t in tensors):
        return False
    from dlgrad_amd.runtime.hip import HIP
    return HIP.DECODE_FUSED


def decode_query_row(x: Tensor, wq: Tensor, wk: Tensor, wv: Tensor, norm, k_store: Tensor, v_store: Tensor,
                     slot: Tensor) -> Tensor | None:
    """Decoding on the hip device with stacked weights: the query projection (1, 1, C) of the single row
    norm(x), while the key and value projections go straight to row (int)slot of the (rows, 1, C) stores --
    project_qkv_row and the store of the two rows as one launch.  None where that is not provided
    (the caller then does the two steps)."""
    if norm is None or norm.weight is None or not _decode_fused(x, wq, k_store, v_store, slot, norm.weight) \
            or not ops.stacked(wq, wk, wv) or x.numel != x.shape[-1]:
        return None
    from dlgrad_amd.runtime.hip import HIP
    C = wq.shape[0]
    w = Buffer(wq.data.ptr, (3 * C, wq.shape[1]), wq.device)
    if k_store.numel != k_store.shape[0] * C or not HIP.decode_qkv_row_fits(x.data, w, norm.weight.data, k_store.data, v_store.data, slot.data):
        return None
    q = x.data.decode_qkv_row(w, norm.weight.data, norm.eps, k_store.data, v_store.data, slot.data)
    return Tensor(q.reshape(x.shape[:-1] + (C,)), requires_grad=False)


def decode_input(wte: Tensor, wpe: Tensor, tok: Tensor, slot: Tensor, T: int, reference_positions: bool):
    """(x, hidden) for one decoding step on the hip device, in one launch: x (1, 1, C) = wte[tok] + wpe[pos]
    with pos = slot (or slot + clamp(slot, 0, 1), the reference's numbering) and hidden (1, T) = arange(T) > slot,
    the cache rows not written yet.  None where not provided."""
    if not _decode_fused(wte, wpe, tok, slot) or wte.ndim != 2 or wpe.ndim != 2 or wte.shape[1] != wpe.shape[1]:
        return None
    x, hidden = Buffer.decode_embed(wte.data, wpe.data, slot.data, T, tok=tok.data, refpos=reference_positions)
    return Tensor(x, requires_grad=False), Tensor(hidden, requires_grad=False)


def decode_window_input(wte: Tensor, wpe: Tensor, seq: Tensor, slot: Tensor, T: int) -> Tensor | None:
    """x (1, T, C) = wte[seq[slot - T + 1 .. slot]] + wpe[0 .. T - 1] on the hip device, in one launch: the
    window of the last T tokens of the (rows, 1) token buffer, embedded.  None where not provided."""
    if not _decode_fused(wte, wpe, seq, slot) or wte.ndim != 2 or wpe.ndim != 2 or wte.shape[1] != wpe.shape[1]:
        return None
    return Tensor(Buffer.decode_embed(wte.data, wpe.data, slot.data, T, seq=seq.data), requires_grad=False)


def decode_append(logits: Tensor, tok: Tensor, slot: Tensor, seq: Tensor) -> bool:
    """seq[slot + 1] = tok = argmax(logits); slot += 1 -- all in place, in one launch, on the hip device.
    False where not provided (nothing done)."""
    if not _decode_fused(logits, tok, slot, seq):
        return False
    logits.data.decode_next_(tok.data, slot.data, seq.data)
    return True


def decode_sample(logits: Tensor, u: Tensor, tok: Tensor, slot: Tensor, seq: Tensor, temperature: float) -> bool:
    """seq[slot + 1] = tok = the token drawn from softmax(logits / temperature) by the uniform number u[slot]
    (inversion of the running sum, as np.random.choice does); slot += 1 -- in place, in one launch, on the hip
    device.  False where not provided (nothing done)."""
    if not _decode_fused(logits, u, tok, slot, seq):
        return False
    logits.data.decode_sample_(u.data, tok.data, slot.data, seq.data, temperature)
    return True


def norm_linear(x: Tensor, norm, weight: Tensor) -> Tensor:
    """norm(x) @ weight^T.  For a single row on the hip device the normalisation happens inside the product
    and the result carries no tape: taken inside nn.inference(), or when neither x nor the weight nor the gain
    requires a gradient; otherwise the two ops (or their one-node form), which record the graph."""
    inside = _row_norm(x, weight.data, norm) if (weight.ndim == 2 and _tape_free(x, weight, norm.weight)) else None
    if inside:
        y = x.data.matmul_nt(weight.data, norm=inside)
        return Tensor(y.reshape(x.shape[:-1] + (weight.shape[0],)), requires_grad=False)
    if ops.tile_norm_applies(x, weight, norm):
        return ops.NormLinearNT.execute(x, weight, norm.weight, eps=norm.eps)
    return norm(x).linear(weight, None)


def mlp_relu(x: Tensor, w_fc: Tensor, w_proj: Tensor, residual: Tensor | None = None, norm=None) -> Tensor:
    """relu(x @ w_fc^T) @ w_proj^T (+ residual): the bias-free feed-forward block of
    examples/gpt.py:69-78.  On the hip device one node whose ReLU, ReLU gradient and residual addition
    happen as the products are stored (ops.MLPRelu); elsewhere the four ops.
    norm: an RMSNorm to apply to x first.  For a single row on the hip device it is applied inside the first
    product, and the result then carries no tape: taken inside nn.inference(), or when no input requires a gradient."""
    if norm is not None:
        inside = _row_norm(x, w_fc.data, norm) if (w_fc.ndim == 2 and w_proj.ndim == 2 and w_proj.device is x.device
                                                   and _tape_free(x, w_fc, w_proj, residual, norm.weight)) else None
        if inside and (residual is None or (residual.device is x.device and residual.shape == x.shape[:-1] + (w_proj.shape[0],))):
            h = x.data.matmul_nt(w_fc.data, epi="relu", norm=inside)
            y = h.matmul_nt(w_proj.data, epi="add", e=residual.data) if residual is not None else h.matmul_nt(w_proj.data)
            return Tensor(y.reshape(x.shape[:-1] + (w_proj.shape[0],)), requires_grad=False)
        if residual is x and ops.use_fused_epilogues(x, w_fc, w_proj) and w_proj.shape[0] == x.shape[-1] and ops.tile_norm_applies(x, w_fc, norm):
            return ops.NormMLPRelu.execute(x, w_fc, w_proj, norm.weight, eps=norm.eps)       # x + mlp(norm(x)) as one node
        x = norm(x)
    if ops.use_fused_epilogues(x, w_fc, w_proj) and (residual is None or (residual.device is x.device and residual.shape == x.shape[:-1] + (w_proj.shape[0],))):
        args = (x, w_fc, w_proj) if residual is None else (x, w_fc, w_proj, residual)
        return ops.MLPRelu.execute(*args)
    out = x.linear(w_fc, None).relu().linear(w_proj, None)
    return out if residual is None else residual + out
