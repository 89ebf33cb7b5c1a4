"""Char-level GPT: the model graph of dlgrad's examples/gpt.py:33-129 on this package's Tensor.

RMSNorm (not LayerNorm), ReLU MLP, no biases, no dropout, untied lm_head, learned
positional embedding -- what that file builds, not what its config comment suggests.
Differences that do not change values: the causal mask (seven small kernels,
examples/gpt.py:52-53) is built once per (T, device) instead of once per block per step,
every parameter is created on the model's device, and the key/value cache of incremental
decoding stays on the device (the reference concatenates it in numpy on the host,
examples/gpt.py:57-60).
"""
from __future__ import annotations

import numpy as np

from dlgrad_amd import Tensor, nn
from dlgrad_amd.helpers import STRICT_REFERENCE, sample_from_logits


def _inference(fn):
    """The decorated method differentiates nothing: it runs inside nn.inference(), where single-row
    products may apply their norm on the way and return results without a tape."""
    import functools

    @functools.wraps(fn)
    def run(*args, **kwargs):
        with nn.inference():
            return fn(*args, **kwargs)
    return run


class GPTConfig:
    def __init__(self, vocab_size: int = 65, block_size: int = 128, n_layer: int = 6, n_head: int = 4,
                 n_embd: int = 128, batch_size: int = 16, learning_rate: float = 1e-4, device: str = "hip") -> None:
        self.vocab_size, self.block_size, self.n_layer = vocab_size, block_size, n_layer
        self.n_head, self.n_embd, self.batch_size = n_head, n_embd, batch_size
        self.learning_rate, self.device = learning_rate, device


class CausalSelfAttention:
    def __init__(self, c: GPTConfig) -> None:
        assert c.n_embd % c.n_head == 0
        self.n_head, self.head_dim = c.n_head, c.n_embd // c.n_head
        self.scale = self.head_dim ** -0.5
        self.q_proj = nn.Linear(c.n_embd, c.n_embd, bias=False, device=c.device)
        self.k_proj = nn.Linear(c.n_embd, c.n_embd, bias=False, device=c.device)
        self.v_proj = nn.Linear(c.n_embd, c.n_embd, bias=False, device=c.device)
        self.c_proj = nn.Linear(c.n_embd, c.n_embd, bias=False, device=c.device)
        # same three parameters, placed back to back so that one product can serve all three projections
        nn.stack_parameters([self.q_proj.weight, self.k_proj.weight, self.v_proj.weight])

    def __call__(self, x: Tensor, cache: "KVCache | None" = None, layer: int = 0,
                 residual: Tensor | None = None, norm=None) -> Tensor:
        """Without a cache, or with an empty one: causal attention over the T positions of x
        (whose k/v projections are stored if a cache is given).  With a filled cache and
        T == 1: the new position attends to everything cached plus itself, no mask
        (examples/gpt.py:44-66).  norm: the RMSNorm to apply to x first (the projections apply it where they can)."""
        T = x.shape[1]
        if cache is None:
            # q, k, v projections, split into heads, ((q @ k^T) * scale).masked_fill(mask, -inf).softmax(dim=3) @ v,
            # merge the heads (examples/gpt.py:45-57): one node on the hip device
            return self.c_proj(nn.self_attention_qkv(x, self.q_proj.weight, self.k_proj.weight, self.v_proj.weight,
                                                     self.n_head, self.scale, norm), residual)
        q_lin, k_lin, v_lin = nn.project_qkv_row(x, self.q_proj.weight, self.k_proj.weight, self.v_proj.weight, norm)   # (B, T, C)
        if cache.length > 0:
            assert T == 1, "incremental attention takes one new position"
            cache.write(layer, k_lin, v_lin, cache.length)
            # the heads of q against the heads of everything cached (examples/gpt.py:58-63)
            y = nn.cached_attention(q_lin, cache.k[layer], cache.v[layer], cache.length + 1, self.n_head, self.scale)
        else:
            cache.write(layer, k_lin, v_lin, 0)               # prefill: the projections are kept for later tokens
            y = nn.causal_self_attention(q_lin, k_lin, v_lin, self.n_head, self.scale)
        return self.c_proj(y, residual)


class KVCache:
    """The k and v projections of every position so far, per layer, on the model's device.

    Stored as (block_size, B, C): the first n positions are then one contiguous view, and
    appending a position is a single device-to-device copy of B*C floats.  nn.cached_attention
    reads the heads of those rows in place: the same (B, h, n, d) values the reference gets by
    concatenating on the host."""

    def __init__(self, c: GPTConfig, batch: int) -> None:
        shape = (c.block_size, batch, c.n_embd)
        self.k = [Tensor.full(shape, 0.0, device=c.device) for _ in range(c.n_layer)]
        self.v = [Tensor.full(shape, 0.0, device=c.device) for _ in range(c.n_layer)]
        self.batch, self.length = batch, 0

    def write(self, layer: int, k: Tensor, v: Tensor, at: int) -> None:
        """k, v: (B, T, C) projections of positions at .. at+T-1."""
        B, T, C = k.shape
        for store, new in ((self.k[layer], k), (self.v[layer], v)):
            rows = new if (B == 1 or T == 1) else new.transpose(0, 1)          # (T, B, C) order
            store[at:at + T].data.copy_(rows.data)


class MLP:
    def __init__(self, c: GPTConfig) -> None:
        self.c_fc = nn.Linear(c.n_embd, 4 * c.n_embd, bias=False, device=c.device)
        self.c_proj = nn.Linear(4 * c.n_embd, c.n_embd, bias=False, device=c.device)

    def __call__(self, x: Tensor, residual: Tensor | None = None, norm=None) -> Tensor:
        """c_proj(relu(c_fc(x))), plus the residual stream if given; norm: the RMSNorm to apply to x first."""
        return nn.mlp_relu(x, self.c_fc.weight, self.c_proj.weight, residual, norm)


class Block:
    def __init__(self, c: GPTConfig) -> None:
        self.ln1 = nn.RMSNorm(c.n_embd, device=c.device)
        self.attn = CausalSelfAttention(c)
        self.ln2 = nn.RMSNorm(c.n_embd, device=c.device)
        self.mlp = MLP(c)

    def __call__(self, x: Tensor, cache: KVCache | None = None, layer: int = 0) -> Tensor:
        x = self.attn(x, cache, layer, residual=x, norm=self.ln1)     # x + attention(norm(x))
        return self.mlp(x, residual=x, norm=self.ln2)                 # x + mlp(norm(x))


_position_ids: dict = {}


def _positions(T: int, device) -> Tensor:
    """0 .. T-1 as a tensor on `device`, made there once per length (the reference builds it anew, and on
    the host, in every forward; examples/gpt.py:96-97)."""
    key = (T, str(device))
    if key not in _position_ids:
        _position_ids[key] = Tensor.arange((T,), device=device)
    return _position_ids[key]


class GPT:
    def __init__(self, c: GPTConfig) -> None:
        self.config = c
        self.wte = nn.Embedding(c.vocab_size, c.n_embd, device=c.device)
        self.wpe = nn.Embedding(c.block_size, c.n_embd, device=c.device)
        self.blocks = [Block(c) for _ in range(c.n_layer)]
        self.ln_f = nn.RMSNorm(c.n_embd, device=c.device)
        self.lm_head = nn.Linear(c.n_embd, c.vocab_size, bias=False, device=c.device)

    def __call__(self, idx: Tensor, targets: Tensor | None = None):
        """idx, targets: (B, T) token ids stored as fp32.  Returns (logits, loss)."""
        B, T = idx.shape
        x = nn.embed_tokens(self.wte, self.wpe, idx, _positions(T, idx.device))
        for block in self.blocks:
            x = block(x)
        logits = nn.norm_linear(x, self.ln_f, self.lm_head.weight)
        if targets is None:
            return logits, None
        V = self.config.vocab_size
        loss = logits.reshape((B * T, V)).cross_entropy_loss(targets.reshape((B * T, 1)))
        return logits, loss

    # ---- incremental decoding with a device-resident key/value cache -----------------------------
    def _hidden(self, idx: Tensor, pos: Tensor, cache: KVCache) -> Tensor:
        x = self.wte(idx) + self.wpe(pos)
        for i, block in enumerate(self.blocks):
            x = block(x, cache, i)
        return self.ln_f(x)

    @_inference
    def prefill(self, idx: Tensor) -> tuple[Tensor, KVCache]:
        """Full forward over idx (B, T) that also fills a fresh cache; returns the logits of
        the last position as (B, 1, V) and the cache (the inference branch of
        examples/gpt.py:103-112, which slices the last position out on the host)."""
        B, T = idx.shape
        cache = KVCache(self.config, B)
        x = self._hidden(idx, _positions(T, idx.device), cache)
        cache.length = T
        C = x.shape[2]
        last = x.reshape((T, C))[T - 1:T] if B == 1 else x.transpose(0, 1)[T - 1:T]
        return self.lm_head(last.reshape((B, 1, C))), cache

    @_inference
    def forward_incremental(self, new_idx: Tensor, pos: Tensor, cache: KVCache) -> Tensor:
        """One new token per sequence: new_idx (B, 1), pos (1, 1) its position id; appends to
        the cache and returns logits (B, 1, V) (examples/gpt.py:114-136)."""
        assert new_idx.shape[1] == 1, "incremental forward expects a single token"
        x = self._hidden(new_idx, pos, cache)
        cache.length += 1
        return self.lm_head(x)

    def generate(self, first_token: int, max_new_tokens: int, temperature: float = 1.0, u=None,
                 reference_positions: bool = STRICT_REFERENCE) -> list[int]:
        """The reference's generate (examples/gpt.py:169-226) with its sampling: the key/value-cache loop of
        generate_greedy_cached, each token drawn on the host from softmax(logits / temperature) of the
        downloaded logits (np.random.choice there; helpers.sample_from_logits here, which is choice() with
        its uniform draw given).  u: max_new_tokens uniform numbers in [0, 1), one per token (a tensor or an
        array); drawn from the device's seeded generator (dlgrad_amd.manual_seed) when None."""
        if u is None:
            u = Tensor.uniform((max(max_new_tokens, 1),), device=self.config.device)
        u = np.asarray(u.numpy() if isinstance(u, Tensor) else u, dtype=np.float32).reshape(-1)
        if u.size < max_new_tokens or not temperature > 0:
            raise ValueError("generate: one uniform number per new token and a positive temperature are needed")
        return self.generate_greedy_cached(first_token, max_new_tokens, reference_positions, (float(temperature), u))

    def generate_greedy_cached(self, first_token: int, max_new_tokens: int,
                               reference_positions: bool = STRICT_REFERENCE, sampling: tuple | None = None) -> list[int]:
        """The control flow of the reference's generate (examples/gpt.py:169-226) with argmax in
        place of sampling (sampling = (temperature, uniform numbers): drawn on the host instead, see
        generate): a full forward when there is no cache, one-token steps after it,
        and -- as there -- no sliding: once the sequence has reached block_size the cache is
        dropped and every further token is a full forward over the last block_size tokens.
        reference_positions reproduces its position id for an incremental token, the sequence
        length *including* that token (one more than the token's index, examples/gpt.py:199).
        Tokens, cache and argmax stay on the device; the ids come back in one download."""
        c = self.config
        seq = Tensor.full((max_new_tokens + 1, 1), float(int(first_token)), device=c.device)
        n, start, cache = 1, 0, None                       # tokens so far; first token of the context window
        for _ in range(max_new_tokens):
            if n - start >= c.block_size:
                start, cache = n - c.block_size, None
            if cache is None:
                logits, cache = self.prefill(seq[start:n].reshape((1, n - start)))
            else:
                length = n - start
                pos = Tensor.full((1, 1), float(length if reference_positions else length - 1), device=c.device)
                logits = self.forward_incremental(seq[n - 1:n], pos, cache)
            if sampling is None:
                nxt = logits.reshape((1, c.vocab_size)).argmax(1)                       # (1, 1), on the device
            else:
                drawn = sample_from_logits(logits.numpy(), sampling[1][n - 1], sampling[0])
                nxt = Tensor(np.array([[drawn]], np.float32), device=c.device)
            seq[n:n + 1].data.copy_(nxt.data)
            n += 1
        return [int(v) for v in seq.numpy().reshape(-1)]

    @_inference
    def generate_greedy(self, first_token: int, max_new_tokens: int) -> list[int]:
        """Greedy decode with full-context recompute per token, context cropped to
        block_size (the loop of examples/gpt.py:231-279 with argmax in place of sampling)."""
        c = self.config
        ids = [int(first_token)]
        for _ in range(max_new_tokens):
            ctx = ids[-c.block_size:]
            T = len(ctx)
            logits, _ = self(Tensor(np.asarray(ctx, dtype=np.float32).reshape(1, T), device=c.device))
            last = logits.reshape((T, c.vocab_size))[T - 1:T]                       # (1, V) view
            ids.append(int(last.argmax(1).numpy()[0, 0]))
        return ids


class StaticDecoder:
    """Greedy decoding as steps of fixed shape, inside the context window and beyond it.

    forward_incremental attends to a cache that grows by one row per token, so every token has
    new tensor shapes and must be issued launch by launch from Python (~130 launches per token
    for the char model, which is what bounds its speed).  Here there are two steps, both of fixed
    shape and without any host input, so each can be captured once as a HIP graph and replayed
    per token:

      step()         while the sequence is shorter than block_size: one new token against the
                     key/value cache.  It always attends to all block_size cache rows and masks
                     the ones not written yet (-inf before the softmax, so they weigh exactly 0).
      step_window()  once block_size tokens exist: the reference keeps no cache from there on
                     (the position embeddings are absolute, so sliding the window by one changes
                     every key and value) and runs the whole model over the last block_size
                     tokens for every new one (examples/gpt.py:176-180, :246-256).  The step
                     gathers that window out of the token buffer at an offset held on the
                     device, runs the full forward and appends the argmax of the last position.

    Everything that changes from token to token -- the token, the cache row to write, the
    position id, the mask, the window offset -- is device data updated by the steps themselves.
    Same tokens as generate_greedy_cached (the probabilities differ only in the order of the
    softmax sums) and, with reference_positions=False, as full recompute (generate_greedy)."""

    def __init__(self, model: GPT, reference_positions: bool = STRICT_REFERENCE, capacity: int | None = None,
                 temperature: float | None = None) -> None:
        """temperature: None decodes greedily; a positive number draws every token from
        softmax(logits / temperature) as the reference's generate does (examples/gpt.py:209-221, :258-266),
        with the uniform numbers of the device's seeded generator (dlgrad_amd.manual_seed), one per token,
        made before the first step (reset) and kept on the device: on the hip device the draw is the last
        launch of the step, so a captured step samples too."""
        c = model.config
        if temperature is not None and not temperature > 0:
            raise ValueError("temperature must be positive")
        self.temperature = None if temperature is None else float(temperature)
        self.model, self.reference_positions = model, reference_positions
        self.capacity = int(capacity) if capacity is not None else 2 * c.block_size + 1     # tokens the buffer holds
        self.cache = KVCache(c, 1)
        self.tok = Tensor.full((1, 1), 0.0, device=c.device)          # token to feed
        self.slot = Tensor.full((1, 1), 0.0, device=c.device)         # its index = cache row to write
        self.seq = Tensor.full((max(self.capacity, c.block_size + 1), 1), 0.0, device=c.device)
        self.u = Tensor.full((self.seq.shape[0],), 0.0, device=c.device) if self.temperature is not None else None
        self.graph = None
        self.window_graph = None

    def reset(self, first_token: int, u=None) -> None:
        """u: the uniform numbers of a sampling decoder, one per token index (a tensor or an array of at least
        as many as will be generated); None draws capacity new ones from the device's generator."""
        if self.u is not None:                                      # in place: captured steps keep reading this address
            if u is None:
                self.u.data.copy_(Tensor.uniform(self.u.shape, device=self.u.device).data)
            else:
                given = np.asarray(u.numpy() if isinstance(u, Tensor) else u, dtype=np.float32).reshape(-1)
                full = np.zeros(self.u.shape, np.float32)
                full[:min(given.size, full.size)] = given[:full.size]
                self.u.data.upload_(full)
        self.tok.data.upload_(np.array([[first_token]], np.float32))
        self.slot.data.upload_(np.zeros((1, 1), np.float32))
        first = np.zeros(self.seq.shape, np.float32)
        first[0, 0] = first_token
        self.seq.data.upload_(first)

    def _attend(self, attn: CausalSelfAttention, x: Tensor, norm, layer: int, hidden: Tensor, residual: Tensor) -> Tensor:
        T = self.model.config.block_size
        q = nn.decode_query_row(x, attn.q_proj.weight, attn.k_proj.weight, attn.v_proj.weight, norm,
                                self.cache.k[layer], self.cache.v[layer], self.slot)     # (k and v go straight to their cache rows)
        if q is None:
            q, k, v = nn.project_qkv_row(x, attn.q_proj.weight, attn.k_proj.weight, attn.v_proj.weight, norm)
            self.cache.k[layer].data.row_store_(k.data, self.slot.data, also=(self.cache.v[layer].data, v.data))
        y = nn.cached_attention(q, self.cache.k[layer], self.cache.v[layer], T, attn.n_head, attn.scale, hidden)
        return attn.c_proj(y, residual)

    def _append(self, logits: Tensor) -> None:
        """logits (1, V) of the newest position: its argmax -- or, for a sampling decoder, the token that u[slot] draws
        from softmax(logits / temperature) -- becomes seq[slot + 1] and the next token; slot advances."""
        if self.temperature is not None:
            if nn.decode_sample(logits, self.u, self.tok, self.slot, self.seq, self.temperature):     # one launch
                return
            # elsewhere as the reference does it: on the host, from the downloaded logits
            s = int(self.slot.numpy()[0, 0])
            drawn = sample_from_logits(logits.numpy(), self.u.numpy().reshape(-1)[s], self.temperature)
            nxt = Tensor(np.array([[drawn]], np.float32), device=logits.device)
        elif nn.decode_append(logits, self.tok, self.slot, self.seq):                   # one launch
            return
        else:
            nxt = logits.argmax(1)                                                      # (1, 1)
        nslot = self.slot + 1.0
        self.seq.data.row_store_(nxt.data, nslot.data)
        self.tok.data.copy_(nxt.data)
        self.slot.data.copy_(nslot.data)

    @_inference
    def step(self) -> None:
        """Feeds self.tok at index self.slot; leaves the argmax in seq[slot + 1] and as the next
        token, and advances slot.  Reads and writes device memory only."""
        m, c = self.model, self.model.config
        slot = self.slot
        got = nn.decode_input(m.wte.weight, m.wpe.weight, self.tok, slot, c.block_size, self.reference_positions)
        if got is not None:
            x, hidden = got
        else:
            # the reference numbers an incremental token one too high (examples/gpt.py:199); token 0 is a full forward there
            pos = slot + slot.clamp(min=0, max=1) if self.reference_positions else slot
            hidden = Tensor.arange((1, c.block_size), device=c.device) > slot               # cache rows not written yet
            x = m.wte(self.tok) + m.wpe(pos)
        for i, block in enumerate(m.blocks):                # each norm is applied by the product that consumes its row
            x = self._attend(block.attn, x, block.ln1, i, hidden, x)
            x = block.mlp(x, x, block.ln2)
        self._append(nn.norm_linear(x, m.ln_f, m.lm_head.weight).reshape((1, c.vocab_size)))

    @_inference
    def step_window(self) -> None:
        """The step for a full window: tokens slot - block_size + 1 .. slot go through the whole model
        at positions 0 .. block_size - 1; the argmax of the last position becomes token slot + 1."""
        m, c = self.model, self.model.config
        T = c.block_size
        x = nn.decode_window_input(m.wte.weight, m.wpe.weight, self.seq, self.slot, T)     # window gathered and embedded in one launch
        if x is None:
            where = Tensor.arange((1, T), device=c.device) + (self.slot - float(T - 1))    # indices into the token buffer
            window = Tensor.embedding(self.seq, where).reshape((1, T))                      # the tokens themselves
            logits, _ = m(window)
        else:
            for block in m.blocks:
                x = block(x)
            logits = nn.norm_linear(x, m.ln_f, m.lm_head.weight)
        self._append(logits.reshape((T, c.vocab_size))[T - 1:T])

    def capture(self) -> None:
        """hip only: records both steps into graphs (one warm-up run of each fixes every address first).
        The warm-up tokens are overwritten by the next reset()."""
        from dlgrad_amd.runtime import hip
        T = self.model.config.block_size
        self.reset(0)
        self.graph = hip.Graph()
        with self.graph.arena():
            self.step()
        with self.graph.capture():
            self.step()
        if self.capacity > T:
            self.slot.data.upload_(np.array([[T - 1]], np.float32))       # a full window, wherever its tokens come from
            self.window_graph = hip.Graph()
            with self.window_graph.arena():
                self.step_window()
            with self.window_graph.capture():
                self.step_window()

    def generate(self, first_token: int, max_new_tokens: int, u=None) -> list[int]:
        """u: for a sampling decoder, the uniform number per token (see reset)."""
        c = self.model.config
        if not 0 <= max_new_tokens <= self.capacity - 1:
            raise ValueError(f"this decoder holds {self.capacity} tokens: at most {self.capacity - 1} new ones")
        self.reset(first_token, u)
        for t in range(max_new_tokens):
            if t < c.block_size - 1:                      # t + 1 tokens so far: still inside the window
                self.graph.replay() if self.graph is not None else self.step()
            else:
                self.window_graph.replay() if self.window_graph is not None else self.step_window()
        return [int(v) for v in self.seq.numpy().reshape(-1)[:max_new_tokens + 1]]

    def close(self) -> None:
        for g in (self.graph, self.window_graph):
            if g is not None:
                g.close()
        self.graph = self.window_graph = None


def init_weights_(model: GPT, seed: int, std: float = 0.02) -> None:
    """Overwrites every parameter with seeded numpy values: N(0, std) for matrices and
    embeddings, ones for the RMSNorm gains -- the same values on any device."""
    rng = np.random.default_rng(seed)
    for name, p in nn.utils.get_state_dict(model).items():
        if ".ln" in f".{name}" and name.endswith("weight"):
            w = np.ones(p.shape, dtype=np.float32)
        else:
            w = (rng.standard_normal(p.shape) * std).astype(np.float32)
        p.data.upload_(w)                                # in place: parameters keep their addresses (and their stacking)
