"""Parts defined by the tests, in plain torch, registered like any other part:
they show that a mixer with state of its own, another feed-forward (also one with
routing), norm, position encoding or whole architecture needs no change to the
package's files.
They are toys, not a model of anyone's."""
import torch

from pytriton_llama_amd.config.registry import register_model
from pytriton_llama_amd.models import CausalLM, LayerCall
from pytriton_llama_amd.parts import (PagedSpec, PagedTensor, ParamSource, Part, StateSpec, WorkList,
                                      build_part, place, register_part)


@register_part("embedding", "toy_embedding")
class ToyEmbedding(Part):
    def __init__(self, vocab_size, hidden_size):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size

    def param_sources(self):
        return [ParamSource("weight", (self.vocab_size, self.hidden_size))]

    def load(self, tensors, dtype, device):
        self.weight = place(tensors["weight"], "matrix", dtype, device)

    def forward(self, ids):
        return self.weight[ids.long()]


@register_part("norm", "toy_meannorm")
class ToyMeanNorm(Part):
    """Subtracts the mean: another norm, with the same interface."""

    def __init__(self, size):
        self.size = size

    def forward(self, x, residual):
        s = x if residual is None else x + residual
        return s - s.mean(-1, keepdim=True), s


@register_part("mixer", "toy_decay_state")
class ToyDecayState(Part):
    """s_t = decay * s_{t-1} + x_t W^T, y_t = s_t: a mixer whose memory is one
    vector per request (no keys, no pages). It starts from the request's state
    slot and writes it back, so any cutting of a sequence gives the same y."""

    graph_capturable = False         # forward reads q_start and the slots on the host

    def __init__(self, hidden_size, decay):
        self.hidden_size, self.decay = hidden_size, decay

    def cache_spec(self):
        return StateSpec((self.hidden_size,), torch.float32)

    def param_sources(self):
        return [ParamSource("w", (self.hidden_size, self.hidden_size))]

    def load(self, tensors, dtype, device):
        self.w = place(tensors["w"], "matrix", dtype, device)

    def forward(self, x, ctx, cache):
        u = (x.float() @ self.w.float().T)
        y = torch.empty_like(u)
        starts = ctx.q_start.tolist()
        slots = ctx.state_slots.tolist()
        for i, slot in enumerate(slots):
            s = cache.state[slot].clone()
            for t in range(starts[i], starts[i + 1]):
                s = self.decay * s + u[t]
                y[t] = s
            if cache.writable:
                cache.state[slot] = s
        return y.to(x.dtype)


@register_part("mixer", "toy_decay_state_on_device")
class ToyDecayStateOnDevice(Part):
    """The same recurrence with a decay rate per channel (a tensor of the checkpoint, drawn
    between 0.5 and 0.9 in the random-weights mode: no norm weight) and without a word from the
    device to the host, so that a step can be recorded as a graph. Where a sequence's rows end is
    read from ctx.q_start on the device: in a recorded step the host's lengths are the upper
    bounds of the step's size class, and rows past the end are padding that must not move the
    state."""

    def __init__(self, hidden_size):
        self.hidden_size = hidden_size

    def cache_spec(self):
        return StateSpec((self.hidden_size,), torch.float32)

    def param_sources(self):
        return [ParamSource("w", (self.hidden_size, self.hidden_size)),
                ParamSource("decay", (self.hidden_size,), "vector", init=("uniform", 0.5, 0.9)),
                ParamSource("bias", (self.hidden_size,), "vector", init=("normal", 0.0, 0.1))]

    def load(self, tensors, dtype, device):
        self.w = place(tensors["w"], "matrix", dtype, device)
        self.decay = place(tensors["decay"], "vector", dtype, device)
        self.bias = place(tensors["bias"], "vector", dtype, device)

    def forward(self, x, ctx, cache):
        u = x.float() @ self.w.float().T + self.bias
        n = ctx.num_seqs
        first, end = ctx.q_start[:n].long(), ctx.q_start[1:n + 1].long()
        slots = ctx.state_slots[:n].long()
        s = cache.state.index_select(0, slots)
        y = torch.zeros_like(u)
        for j in range(ctx.max_q_len):
            row = first + j
            live = (row < end)[:, None]
            row = torch.where(live[:, 0], row, first)          # rows past the end: a row of its own
            s = torch.where(live, self.decay * s + u.index_select(0, row), s)
            y.index_copy_(0, row, torch.where(live, s, y.index_select(0, row)))
        if cache.writable:
            cache.state.index_copy_(0, slots, s)
        return y.to(x.dtype)


@register_part("mixer", "toy_chunked_decay")
class ToyChunkedDecay(Part):
    """The recurrence of ToyDecayState, s_t = decay * s_{t-1} + x_t W^T, y_t = s_t, worked out
    block by block: the part asks the engine for a list that cuts the rows of a step into
    blocks of 32 (another tiling than any kernel of the package has) and computes every block
    of the list on its own, from the state at the start of the step and all rows of the
    sequence up to the block's. Rows that no item of the list covers would stay zero. Nothing
    is read on the host, so its steps are recorded as graphs, where the list is as long as the
    size class can need and ends in empty items."""
    BLOCKS = WorkList(32)

    def __init__(self, hidden_size, decay):
        self.hidden_size, self.decay = hidden_size, decay

    def work_lists(self):
        return (self.BLOCKS,)

    def cache_spec(self):
        return StateSpec((self.hidden_size,), torch.float32)

    def param_sources(self):
        return [ParamSource("w", (self.hidden_size, self.hidden_size))]

    def load(self, tensors, dtype, device):
        self.w = place(tensors["w"], "matrix", dtype, device)

    def forward(self, x, ctx, cache):
        u = x.float() @ self.w.float().T                                 # [T, H]
        T, n = u.shape[0], ctx.num_seqs
        seq, off = (t.long() for t in ctx.work[self.BLOCKS])            # [W] each
        q_start = ctx.q_start.long()
        first, end = q_start[seq], q_start[seq + 1]
        rows = (first + off)[:, None] + torch.arange(32, device=u.device)[None, :]       # [W, 32]
        live = rows < end[:, None]                                       # an empty item: no row
        t = torch.arange(T, device=u.device)
        dist = rows[:, :, None] - t[None, None, :]                       # [W, 32, T]
        counts = (t[None, None, :] >= first[:, None, None]) & (dist >= 0) & live[:, :, None]
        weights = torch.where(counts, torch.pow(self.decay, dist.clamp(min=0).float()),
                              torch.zeros((), device=u.device))
        y_blocks = torch.einsum("wat,th->wah", weights, u)
        s0 = cache.state.index_select(0, ctx.state_slots.long()[seq])   # the state the step starts from
        since = (rows - first[:, None] + 1).clamp(min=0).float()
        y_blocks = y_blocks + torch.pow(self.decay, since)[:, :, None] * s0[:, None, :]
        y = torch.zeros((T + 1, u.shape[1]), dtype=torch.float32, device=u.device)
        # rows without a sequence go to a row of their own behind the last, which is dropped
        y.index_copy_(0, torch.where(live, rows, torch.full_like(rows, T)).flatten(), y_blocks.flatten(0, 1))
        if cache.writable:
            # a sequence's new state is its last row's (a place without rows names the padding
            # slot and writes there what nobody reads)
            last = (q_start[1:n + 1] - 1).clamp(min=0)
            cache.state.index_copy_(0, ctx.state_slots.long()[:n], y.index_select(0, last))
        return y[:T].to(x.dtype)


@register_part("mixer", "toy_latent_memory")
class ToyLatentMemory(Part):
    """A mixer whose paged memory is one tensor a token, not keys and values: it keeps
    c_t = x_t Wc^T (``latent`` numbers) of every token in pages and a token reads all of them
    up to its own, y_t = (sum_s p_ts c_s) Wo^T with p_t = softmax_s((x_t Wq^T) . c_s / sqrt(latent))."""
    graph_capturable = False         # forward reads the tables on the host

    def __init__(self, hidden_size, latent):
        self.hidden_size, self.latent = hidden_size, latent

    def cache_spec(self):
        return PagedSpec((PagedTensor("latent", (self.latent,)),))

    def param_sources(self):
        H, L = self.hidden_size, self.latent
        return [ParamSource("wc", (L, H)), ParamSource("wq", (L, H)), ParamSource("wo", (H, L))]

    def load(self, tensors, dtype, device):
        self.wc, self.wq, self.wo = (place(tensors[n], "matrix", dtype, device) for n in ("wc", "wq", "wo"))

    def forward(self, x, ctx, cache):
        L, P = self.latent, cache.page_size
        group = ctx.groups[cache.group]
        pool = cache.latent                                              # [pages, page_size, latent]
        assert pool.shape[1:] == (P, L) and set(cache.tensors) == {"latent"}
        c = x.float() @ self.wc.float().T
        q = x.float() @ self.wq.float().T
        if cache.writable:
            pool.view(-1, L).index_copy_(0, group.slots.long(), c.to(pool.dtype))
        starts, lens, tables = ctx.q_start.tolist(), ctx.ctx_len.tolist(), group.block_table.tolist()
        y = torch.empty_like(c)
        for i in range(ctx.num_seqs):
            n, rows = lens[i], q[starts[i]:starts[i + 1]]
            pages = torch.tensor(tables[i][:-(-n // P)], device=x.device)
            memory = pool.index_select(0, pages).reshape(-1, L)[:n].float()
            position = torch.arange(n - rows.shape[0], n, device=x.device)
            scores = rows @ memory.T / L ** 0.5
            scores = scores.masked_fill(torch.arange(n, device=x.device)[None, :] > position[:, None], float("-inf"))
            y[starts[i]:starts[i + 1]] = torch.softmax(scores, dim=-1) @ memory
        return (y @ self.wo.float().T).to(x.dtype)


@register_part("feed_forward", "toy_relu")
class ToyRelu(Part):
    def __init__(self, hidden_size, inner):
        self.hidden_size, self.inner = hidden_size, inner

    def param_sources(self):
        return [ParamSource("w1", (self.inner, self.hidden_size)),
                ParamSource("w2", (self.hidden_size, self.inner))]

    def load(self, tensors, dtype, device):
        self.w1 = place(tensors["w1"], "matrix", dtype, device)
        self.w2 = place(tensors["w2"], "matrix", dtype, device)

    def forward(self, x):
        return torch.relu(x @ self.w1.T) @ self.w2.T


@register_part("feed_forward", "toy_routed")
class ToyRouted(Part):
    """A feed-forward with routing: router logits in float32, the two best experts of every
    token, their outputs mixed by the softmax over the two logits. Experts are small ReLU
    networks kept in one stacked tensor."""
    graph_capturable = False         # the rows of an expert are counted on the host

    def __init__(self, hidden_size, inner, experts):
        self.hidden_size, self.inner, self.experts = hidden_size, inner, experts

    def param_sources(self):
        E, H, I = self.experts, self.hidden_size, self.inner
        return [ParamSource("router", (E, H)), ParamSource("w1", (E * I, H)),
                ParamSource("w2", (E * H, I))]

    def load(self, tensors, dtype, device):
        E, H, I = self.experts, self.hidden_size, self.inner
        self.router = place(tensors["router"], "matrix", dtype, device).float()
        self.w1 = place(tensors["w1"], "matrix", dtype, device).view(E, I, H)
        self.w2 = place(tensors["w2"], "matrix", dtype, device).view(E, H, I)

    def forward(self, x):
        logits = x.float() @ self.router.T                                   # [T, E]
        top, idx = logits.topk(2, dim=-1)
        mix = torch.softmax(top, dim=-1)
        y = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        for e in range(self.experts):
            for slot in range(2):
                rows = (idx[:, slot] == e).nonzero().flatten()
                if rows.numel():
                    xe = x[rows].float()
                    ye = torch.relu(xe @ self.w1[e].float().T) @ self.w2[e].float().T
                    y[rows] += mix[rows, slot, None] * ye
        return y.to(x.dtype)


@register_part("position", "toy_decay")
class ToyDecayPosition(Part):
    """Another position encoding, not a rotation: q is multiplied by g_j ** p and k by
    g_j ** -p (g_j a little below 1, one per element of the head), so a score depends on the
    distance of the two positions only and far keys fade. It takes the path of position parts
    that are not rotary: ``rotary_inv_freq`` is None and ``apply`` changes q and k in place."""

    def __init__(self, head_dim, strength):
        self.head_dim, self.strength = head_dim, strength
        self.log_g = -strength * torch.arange(1, head_dim + 1, dtype=torch.float32) / head_dim

    def load(self, tensors, dtype, device):
        self.log_g_dev = self.log_g.to(device)

    def rotary_inv_freq(self):
        return None

    def apply(self, q, k, positions):
        f = torch.exp(positions.float()[:, None, None] * self.log_g_dev[None, None, :])
        q.copy_((q.float() * f).to(q.dtype))
        k.copy_((k.float() / f).to(k.dtype))


@register_part("head", "toy_head")
class ToyHead(Part):
    def __init__(self, vocab_size, hidden_size):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size

    def param_sources(self):
        return [ParamSource("weight", (self.vocab_size, self.hidden_size))]

    def load(self, tensors, dtype, device):
        self.weight = place(tensors["weight"], "matrix", dtype, device)

    def forward(self, x):
        return x.float() @ self.weight.float().T


class ToyConfig:
    def __init__(self, d):
        self.__dict__.update(d)
        self.initializer_range = d.get("initializer_range", 0.3)

    @classmethod
    def from_dict(cls, d):
        return cls(d)


def build_toy(cfg: ToyConfig) -> CausalLM:
    """layers: list of "state" / "attention" names; the run order is given by the
    config too (it may name a layer twice)."""
    H, V = cfg.hidden_size, cfg.vocab_size
    emb = build_part("embedding", "toy_embedding", vocab_size=V, hidden_size=H)
    blocks, prefixes = [], [("emb.", emb)]
    for i, kind in enumerate(cfg.layers):
        if kind == "state":
            mixer = build_part("mixer", "toy_decay_state", hidden_size=H, decay=cfg.decay)
        elif kind == "state_on_device":
            mixer = build_part("mixer", "toy_decay_state_on_device", hidden_size=H)
        elif kind == "chunked":
            mixer = build_part("mixer", "toy_chunked_decay", hidden_size=H, decay=cfg.decay)
        elif kind == "latent":
            mixer = build_part("mixer", "toy_latent_memory", hidden_size=H, latent=cfg.latent)
        else:
            if getattr(cfg, "toy_position", False):
                pos = build_part("position", "toy_decay", head_dim=cfg.head_dim, strength=0.02)
            else:
                pos = build_part("position", "rotary", head_dim=cfg.head_dim, theta=100.0)
            mixer = build_part("mixer", "paged_attention", hidden_size=H, num_heads=cfg.heads,
                               num_kv_heads=cfg.kv_heads, head_dim=cfg.head_dim, position=pos,
                               window=getattr(cfg, "window", None))
        norm_name, norm_kw = (("toy_meannorm", dict(size=H)) if cfg.toy_norm
                              else ("rmsnorm", dict(size=H, eps=1e-5)))
        if getattr(cfg, "experts", 0):
            ffn = build_part("feed_forward", "toy_routed", hidden_size=H, inner=cfg.inner,
                             experts=cfg.experts)
        elif cfg.toy_ffn:
            ffn = build_part("feed_forward", "toy_relu", hidden_size=H, inner=cfg.inner)
        else:
            ffn = build_part("feed_forward", "swiglu", hidden_size=H, intermediate_size=cfg.inner)
        b = build_part("block", "prenorm", input_norm=build_part("norm", norm_name, **norm_kw),
                       mixer=mixer, post_norm=build_part("norm", norm_name, **norm_kw), feed_forward=ffn)
        blocks.append(b)
        for role, part in b.children().items():
            prefixes.append((f"l{i}.{role}.", part))
    final = build_part("norm", "toy_meannorm", size=H) if cfg.toy_norm else \
        build_part("norm", "rmsnorm", size=H, eps=1e-5)
    head = build_part("head", "toy_head", vocab_size=V, hidden_size=H)
    prefixes += [("final.", final), ("head.", head)]
    order = getattr(cfg, "order", None) or list(range(len(blocks)))
    # every call gets a cache layer of its own, so a block that runs twice keeps two memories
    cache_layers = [blocks[b].cache_spec() for b in order]
    schedule = [LayerCall(b, i) for i, b in enumerate(order)]
    return CausalLM(cfg, emb, blocks, final, head, cache_layers, schedule, prefixes)


register_model("ToyStateLM", ToyConfig, build_toy)


def toy_plain_forward(model, token_ids):
    """Whole-sequence logits of an all-toy model (state mixers only), no cache."""
    x = model.embedding.weight[torch.as_tensor(token_ids)].float()
    h, residual = x, None
    for call in model.schedule:
        b = model.blocks[call.block]
        h, residual = b.input_norm.forward(h, residual)
        u = h @ b.mixer.w.float().T
        s = torch.zeros(u.shape[1])
        ys = []
        for t in range(u.shape[0]):
            s = b.mixer.decay * s + u[t]
            ys.append(s)
        h = torch.stack(ys)
        h, residual = b.post_norm.forward(h, residual)
        h = b.feed_forward.forward(h)
    h, _ = model.final_norm.forward(h, residual)
    return model.head.forward(h)
