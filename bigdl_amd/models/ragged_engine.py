"""Ragged engine: decoder stacks whose layers are not all alike, stepped over a flat batch of token rows.

``NativeDecoder`` runs families whose layers share one shape on a slot cache in fp16.  Designs that interleave kinds of
token mixers (windowed attention with kept first tokens, score maps that are subtracted, layers that read another
layer's keys and values, gated linear recurrences), that keep the residual stream in 32 bits, or that want prompts cut
into arbitrary portions next to single decoded tokens run here instead:

* a step takes ``[(slot, token ids), ...]``: any mix of prompt portions and single tokens, one row per token.  Every
  product runs once over all rows; the mixers read ``BatchMeta`` (row -> sequence, position, pages);
* keys / values live in 64-token pages of a ``PagedStatePool``, per-sequence state in its slots;
* the mixers are described by small dataclasses whose fields are the design's constants, so a new design is a new list
  of them (``models/lipizen.py``, ``models/merusun.py``, ``models/filanex.py`` and ``models/dimelix.py`` build one from
  a ``config.json``);
* four residual forms: the post-sum norm x <- norm(alpha x + f(x)), the sandwich x <- x + norm_b(f(norm_a(x))), the
  parallel pre-norm block u = norm(x), x <- x + mixer(u) + ff(u), and the sequential pre-norm block x <- x + f(norm(x))
  per sublayer, whose stream may be kept in several copies that every sublayer reads and rewrites with learned weights;
* a run of layers may be executed several times with the same weights (every execution has its own cache), with the
  embedding output mixed back into the stream in front of a pass; the embedding may add a row of a token-pair table;
* matrix products are the library's (bf16 inputs with 32-bit accumulation, or plain float32), everything between them
  is ``ops/ragged.py``.
"""
from __future__ import annotations

import math
import os
import time
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import torch
import torch.nn.functional as F

from ..ops import ragged as R
from .paged import PagedStatePool


@dataclass
class WindowAttention:
    """Softmax attention over cache pages.  ``maps`` = 2: two score maps per head (queries / keys are [map 1 | map 2])
    over the same values, combined as a1 - lam * a2 (differential attention)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    maps: int = 1
    lam: float = 0.0               # weight of the second map
    out_scale: float = 1.0         # after the per-head output norm
    out_norm: bool = False         # each head's output divided by its root mean square (no weight)
    conv_taps: int = 0             # short causal convolution behind the q / k / v projections (0: none)
    qk_norm: bool = False          # RMS norm over ``dim`` with a weight shared by heads and maps, before rotation
    rot_dims: int = 0              # leading channels of every map that are rotated (pairs i, i + rot_dims / 2)
    rot_base: float = 10000.0
    rot_factor: float = 1.0        # linear scaling: frequencies divided by this
    window: int = 0                # 0: full causal attention
    keep_first: int = 0            # the first tokens stay visible behind the window
    gate: bool = False             # one sigmoid gate per head, from the mixer's input
    kv_from: Optional[int] = None  # read this layer's cache instead of projecting keys / values
    bias: bool = False             # the q / k / v projections have biases
    sink: Optional[float] = None   # score of a key without a value that every query sees: exp(sink) joins the normaliser
    chunk: int = 0                 # > 0: keys are visible only inside the query's block of this many positions (from position 0)
    softcap: float = 0.0           # > 0: score <- softcap * tanh(score / softcap), after the scale
    rot_neighbours: bool = False   # rotated pairs are (2 i, 2 i + 1) instead of (i, i + rot_dims / 2)
    rot_freqs: Optional[tuple] = None  # the pairs' frequencies, if they are not base^(-2 i / rot_dims) / rot_factor
    rot_amp: float = 1.0           # cosine and sine are multiplied by this
    gate_channels: bool = False    # with ``gate``: one sigmoid gate per output channel instead of one per head
    head_sinks: bool = False       # every head has a learned sink score (``LayerTensors.sinks``) instead of the one number ``sink``
    dist_slopes: Optional[tuple] = None  # per head: slope * (i - j) is taken off the scaled score of query i and key j
    v_from_k: bool = False         # no value projection: the values are the key projections as they are before norm and rotation


@dataclass
class LatentAttention:
    """Attention over a compressed cache.  Per token one latent row c (``rank`` channels, RMS-normed with a weight) and
    one rotated key part (``rot_dim`` channels) shared by all heads are kept; head h's keys are [W_uk,h c | rotated part],
    its values W_uv,h c.  The engine folds W_uk into the queries and W_uv behind the weighted sum, so the kernel sees one
    key/value head with key rows [c | rotated part] whose values are the rows' leading ``rank`` channels."""
    heads: int
    dim: int                       # unrotated channels of a head's queries and keys
    rot_dim: int                   # rotated channels, after the unrotated ones
    vdim: int
    rank: int
    scale: float
    rot_dims: int = 0              # leading channels of the rotated part that turn (neighbouring pairs 2 i, 2 i + 1)
    rot_base: float = 10000.0
    window: int = 0
    gate: bool = False             # one sigmoid gate per output channel, from the mixer's input, behind the value up-projection
    out_scale: float = 1.0


@dataclass
class DeltaRule:
    """Generalised delta rule with a matrix state per head (keys, values and receptance of ``dim`` channels each):
    S <- diag(w) S - (a * n)(n^T S) + k v^T with the unit key n = k / sqrt(|k|^2 + unit_eps), both terms reading the old state;
    o = S^T r.  The decay w = exp(-decay_rate * sigmoid(W_2 tanh(W_1 h) + b_w)) comes through a low-rank pair of products,
    the removal rate a = sigmoid(W_a h + b_a); both are per head and key channel.  Each head's output is divided by its
    root mean square, weighted, gated by a sigmoid of a projection of the mixer's input and multiplied by ``out_scale``."""
    heads: int
    dim: int
    decay_rank: int
    decay_rate: float = math.exp(-0.5)
    unit_eps: float = 1e-6
    out_scale: float = 1.0


@dataclass
class SideBySide:
    """Two mixers that read the same input; their outputs are summed, each with its own weight (carried by the mixers'
    ``out_scale``, so that one output projection [W_left | W_right] serves both).  The two must keep different kinds of
    state (pages against a matrix), since an execution has one cache of each kind."""
    left: object
    right: object


@dataclass
class Hgrn2:
    """Gated linear recurrence with a matrix state per head: S <- diag(f) S + (1 - f) v^T, o = S^T q."""
    heads: int
    dim: int
    vdim: int


@dataclass
class Mlstm:
    """Matrix memory with exponential gates held stable by a running maximum m (all per head, log gates i and f):
    m' = max(f + m, i), S' = e^(f + m - m') S + e^(i - m') k v^T, n' likewise with k, o = S'^T q / (max(|n' . q|, e^-m') + tiny),
    q scaled by dim^-1/2; gates are soft-capped, log f = logsigmoid(.).  Each head's output is divided by its root mean
    square, weighted, and gated by a sigmoid of a projection of the mixer's input."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float
    m_start: float = 0.0
    den_floor: float = 1e-6


@dataclass
class ClampedGlu:
    """g = min(gate, limit), u = clamp(up, -limit, limit), y = g * sigmoid(slope * g) * (u + 1)"""
    ff: int
    limit: float
    slope: float = 1.702


@dataclass
class RoutedExperts:
    """Mixture of small experts.  ``act`` "relu2": y = W_down relu(W_up h)^2; "swiglu": y = W_down (silu(W_gate h) * W_up h)
    (``LayerTensors.w_up`` then holds the gate and up rows of an inner channel next to each other).  Scores are a softmax
    over all experts' router logits or a sigmoid per expert (32-bit); experts come in ``groups`` equal runs of neighbours,
    a group scores as the sum of its ``group_top`` best experts, and the ``top`` best experts inside the ``keep`` best
    groups are used, weighted by score * ``scale``, the scores first divided by their sum (+ 1e-20) with ``renorm``.
    ``shared_ff`` > 0: one more expert of that inner size that every token uses with weight 1."""
    experts: int
    top: int
    ff: int
    groups: int = 1
    keep: int = 1
    scale: float = 1.0
    shared_ff: int = 0
    score: str = "softmax"         # or "sigmoid"
    group_top: int = 1
    renorm: bool = False
    act: str = "relu2"             # or "swiglu"


@dataclass
class DenseMlp:
    """y = W_down act(W_up h + b_up) + b_down, act "gelu_erf" (0.5 z (1 + erf(z / sqrt 2))), "gelu_tanh", "relu2" or "xielu"
    (a z^2 + z / 2 right of zero, (1/2 + b)(e^z - 1 - z) + z / 2 left of it, a and b = softplus of two learned numbers of the
    layer, ``LayerTensors.act_params``).  In the parallel block its up projection is stacked behind the mixer's input
    projections (one product reads the normed stream once)."""
    ff: int
    act: str = "gelu_erf"
    bias: bool = True


@dataclass
class PairEmbedding:
    """A second embedding table indexed by a hash of (previous token, token): row (prev * mul_prev + cur * mul_cur) mod
    buckets; a sequence's first token, which has no previous one, takes row ``buckets`` (the table's last)."""
    buckets: int
    mul_prev: int
    mul_cur: int

    def rows(self, prev: int, tokens: Sequence[int]) -> List[int]:
        """``prev``: the sequence's last token so far, -1 for a new sequence"""
        out = []
        for t in tokens:
            out.append(self.buckets if prev < 0 else (prev * self.mul_prev + int(t) * self.mul_cur) % self.buckets)
            prev = int(t)
        return out


@dataclass
class RaggedConfig:
    vocab: int
    width: int
    mixers: list                   # one mixer dataclass per layer
    mlps: list                     # ClampedGlu or None per layer
    norm_eps: float = 1e-6
    norm_groups: int = 1
    residual_alpha: float = 1.0    # x <- norm(alpha * x + sublayer(x))
    logit_softcap: float = 0.0
    name: str = "ragged"
    embed_scale: float = 1.0
    block: str = "post_sum"        # "post_sum": x <- norm(alpha x + f(x)); "sandwich": x <- x + norm_b(f(norm_a(x)));
                                   # "parallel": u = norm(x), x <- x + mixer(u) + ff(u); "pre_norm": x <- x + f(norm(x)) per sublayer
    streams: int = 1               # "pre_norm": copies of the stream; every sublayer reads a weighted sum of them and writes
                                   # X[t] <- sum_s mix[s, t] X[s] + out[t] f(.) (``LayerTensors.hc1 / hc2``); the model's output is their sum
    runs: Optional[list] = None    # layer index of every layer execution, in order (None: every layer once); an execution
                                   # has its own cache / state, whatever weights it shares
    mix_in: tuple = ()             # executions in front of which x <- W_mix [x ; embedding output]
    pair_embed: Optional[PairEmbedding] = None

    def layer_runs(self) -> list:
        return list(range(len(self.mixers))) if self.runs is None else list(self.runs)


@dataclass
class LayerTensors:
    w_in: torch.Tensor                       # stacked input projections [rows, width], activation type
    w_out: torch.Tensor
    norm1: torch.Tensor
    norm2: Optional[torch.Tensor] = None
    conv_w: Optional[torch.Tensor] = None    # float [convolved channels, taps]
    q_norm: Optional[torch.Tensor] = None
    k_norm: Optional[torch.Tensor] = None
    inv_freq: Optional[torch.Tensor] = None
    f_bias: Optional[torch.Tensor] = None
    lower: Optional[torch.Tensor] = None
    o_norm: Optional[torch.Tensor] = None
    w_gu: Optional[torch.Tensor] = None      # [gate; up]
    w_down: Optional[torch.Tensor] = None
    b_in: Optional[torch.Tensor] = None      # biases of the stacked input projections (zeros where there is none)
    norm1b: Optional[torch.Tensor] = None    # sandwich form: norms behind the mixer and the feed-forward
    norm2b: Optional[torch.Tensor] = None
    w_uk: Optional[torch.Tensor] = None      # latent attention: [heads, dim, rank] and [heads, vdim, rank]
    w_uv: Optional[torch.Tensor] = None
    gate_bias: Optional[torch.Tensor] = None  # mLSTM: float [2 heads], input gates then forget gates
    w_router: Optional[torch.Tensor] = None  # float [experts, width]
    w_up: Optional[torch.Tensor] = None      # [experts, ff, width]
    w_dn: Optional[torch.Tensor] = None      # [experts, width, ff]
    w_sup: Optional[torch.Tensor] = None     # shared expert
    w_sdn: Optional[torch.Tensor] = None
    b_down: Optional[torch.Tensor] = None    # dense feed-forward: bias of the down projection (the up bias is part of b_in)
    w_ff: Optional[torch.Tensor] = None      # dense feed-forward of the sequential pre-norm block: its up projection
    act_params: Optional[tuple] = None       # the two curvatures of an "xielu" feed-forward (floats, softplus already applied)
    sinks: Optional[torch.Tensor] = None     # float [heads]: learned sink scores
    slopes: Optional[torch.Tensor] = None    # float [heads]: distance slopes
    hc1: Optional[torch.Tensor] = None       # float [2 S + S S]: read-out, write-back and mixing weights of the stream copies
    hc2: Optional[torch.Tensor] = None       # around the mixer (hc1) and the feed-forward (hc2)
    w_decay: Optional[torch.Tensor] = None   # delta rule: second product of the decay's low-rank pair [heads dim, rank]
    decay_bias: Optional[torch.Tensor] = None  # float [heads dim]
    remove_bias: Optional[torch.Tensor] = None  # float [heads dim]
    left: Optional["LayerTensors"] = None    # side-by-side mixers: what each of the two needs beyond the shared projections
    right: Optional["LayerTensors"] = None


def rotary_inv_freq(dims: int, base: float, factor: float) -> torch.Tensor:
    """f_i = base^(-2 i / dims) / factor, i < dims / 2, evaluated in float32"""
    i = torch.arange(dims // 2, dtype=torch.float32)
    return (float(base) ** (-2.0 * i / dims)) / float(factor)


def yarn_inv_freq(dims: int, base: float, factor: float, original: float, fast: float, slow: float):
    """Frequencies of a rotation stretched for contexts longer than the ``original`` one, pair by pair: with
    index(t) = dims ln(original / (2 pi t)) / (2 ln base) the pair whose wavelength turns t times in the original context,
    lo = max(floor(index(fast)), 0), hi = min(ceil(index(slow)), dims - 1) and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
    f_i' = r_i f_i / factor + (1 - r_i) f_i: fast pairs keep their frequency, slow ones are divided by ``factor``.
    Returns (float32 frequencies, amplitude 0.1 ln(factor) + 1 that multiplies cosine and sine)."""
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]

    def index(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo, hi = max(math.floor(index(fast)), 0), min(math.ceil(index(slow)), dims - 1)
    out = []
    for i, fi in enumerate(f):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * r + fi * (1.0 - r))
    return torch.tensor(out, dtype=torch.float64).to(torch.float32), 0.1 * math.log(factor) + 1.0


class RaggedDecoder:
    ragged = True                  # serving/continuous.py steps such an engine with mixed batches

    def __init__(self, cfg: RaggedConfig, embed: torch.Tensor, layers: List[LayerTensors], final_norm: torch.Tensor,
                 head: torch.Tensor, act_dtype=torch.bfloat16, device="cuda", pair_table: Optional[torch.Tensor] = None,
                 w_mix: Optional[torch.Tensor] = None):
        """``pair_table`` [buckets + 1, width]: the token-pair embedding of ``cfg.pair_embed``; ``w_mix`` [width, 2 width]:
        the projection of [stream ; embedding output] in front of the executions named in ``cfg.mix_in``."""
        self.cfg, self.embed, self.layers, self.final_norm, self.head = cfg, embed, layers, final_norm, head
        self.pair_table, self.w_mix = pair_table, w_mix
        self.act = act_dtype
        self.device = torch.device(device)
        self.ops = R.ops_for(self.device)
        self.pool: Optional[PagedStatePool] = None
        self.runs = cfg.layer_runs()
        if any(not 0 <= li < len(layers) for li in self.runs) or any(not 0 <= ri < len(self.runs) for ri in cfg.mix_in):
            raise ValueError("layer executions outside the layer list")
        if cfg.mix_in and (w_mix is None or tuple(w_mix.shape) != (cfg.width, 2 * cfg.width) or cfg.block != "parallel"):
            raise ValueError("mixing the embedding output back in needs a [width, 2 width] projection and the parallel block")
        if cfg.pair_embed is not None and (pair_table is None or tuple(pair_table.shape) != (cfg.pair_embed.buckets + 1, cfg.width)):
            raise ValueError("the token-pair table must have buckets + 1 rows of the stream's width")
        self._kv_run = {}                  # execution -> the execution whose cache it reads (itself unless kv_from is set)
        latest = {}
        for ri, li in enumerate(self.runs):
            m = cfg.mixers[li]
            self._kv_run[ri] = ri
            if isinstance(m, WindowAttention) and m.kv_from is not None:
                o = cfg.mixers[m.kv_from] if 0 <= m.kv_from < len(cfg.mixers) and m.kv_from in latest else None
                if not isinstance(o, WindowAttention) or o.kv_from is not None or \
                        (o.kv_heads, o.dim, o.vdim, o.maps) != (m.kv_heads, m.dim, m.vdim, m.maps):
                    raise ValueError(f"layer {li}: kv_from must name an earlier attention layer with keys of its own and "
                                     "the same head layout")
                self._kv_run[ri] = latest[m.kv_from]
            latest[li] = ri
        if cfg.block == "pre_norm":
            S = cfg.streams
            if not 1 <= S <= 8:
                raise ValueError("1 to 8 copies of the stream")
            # read-out weights that sum the copies (the model's output), and the coefficients of a plain residual sum
            self._sum_read = torch.cat([torch.ones(2 * S), torch.eye(S).reshape(-1)]).to(self.device)
            for lt, mlp in zip(layers, cfg.mlps):
                for name in ("hc1", "hc2") if mlp is not None else ("hc1",):
                    if getattr(lt, name) is None:
                        if S != 1:
                            raise ValueError("several copies of the stream need every sublayer's coefficients")
                        setattr(lt, name, self._sum_read)
        self.first_cost = self.rest_cost_mean = self.peak_memory = 0.0
        # BIGDL_RAGGED_GRAPH=1: steps that carry one token per sequence are recorded once per (sequences, page-table
        # width) and replayed as one hipGraph.  Off by default: every step is issued kernel by kernel.  With recording
        # on, a replay of a long trace ended with the GPU in a fault that has no established cause yet.
        self.use_graph = self.device.type == "cuda" and os.environ.get("BIGDL_RAGGED_GRAPH", "0") == "1"
        self._graphs = {}
        self.graph_replays = 0

    # ------------------------------------------------------------------ state
    def state_specs(self):
        """what every layer execution keeps, by execution index"""
        specs = {}
        for ri, li in enumerate(self.runs):
            top = self.cfg.mixers[li]
            s = []
            for m in ((top.left, top.right) if isinstance(top, SideBySide) else (top,)):
                s += self._mixer_specs(m)
            kinds = [spec[0] if spec[0] != "kv" else "k" for spec in s]
            if len(set(kinds)) != len(kinds):
                raise ValueError(f"layer {li}: mixers side by side must keep different kinds of state")
            specs[ri] = s
        return specs

    def _mixer_specs(self, m):
        s = []
        if isinstance(m, WindowAttention):
            if m.kv_from is None:
                s.append(("kv", m.kv_heads, m.maps * m.dim, m.vdim))
            if m.conv_taps > 1:
                s.append(("tail", m.conv_taps - 1, self._conv_channels(m)))
        elif isinstance(m, LatentAttention):
            s.append(("k", 1, m.rank + m.rot_dim))          # values are the rows' leading channels
        elif isinstance(m, Hgrn2):
            s.append(("matrix", m.heads, m.dim, m.vdim))
        elif isinstance(m, Mlstm):
            s.append(("matrix", m.heads, m.dim, m.vdim + 1))  # S and, as its last column, the normaliser n
            s.append(("vector", m.heads))                   # the running maximum of every head
        elif isinstance(m, DeltaRule):
            s.append(("matrix", m.heads, m.dim, m.dim))
        return s

    @staticmethod
    def _conv_channels(m: WindowAttention) -> int:
        c = m.heads * m.maps * m.dim
        if m.kv_from is None:
            c += m.kv_heads * (m.maps * m.dim + (0 if m.v_from_k else m.vdim))
        return c

    def ensure_pool(self, max_tokens: int, slots: int) -> PagedStatePool:
        p = self.pool
        if p is None or p.num_pages * R.PAGE < max_tokens or p.slots < slots or p.len_of:
            self.pool = PagedStatePool(self.state_specs(), max_tokens, slots, self.act, self.device)
            self._graphs.clear()              # recorded steps hold the old pool's addresses
        return self.pool

    # ------------------------------------------------------------------ layers
    def _attention(self, li, m: WindowAttention, lt: LayerTensors, P, meta):
        """``li`` (here and in the other mixers): the execution's index, which names its cache / state in the pool"""
        ops, pool, eps = self.ops, self.pool, self.cfg.norm_eps
        turn = dict(interleaved=m.rot_neighbours, rot_amp=m.rot_amp)
        cq = m.heads * m.maps * m.dim
        ck = m.kv_heads * m.maps * m.dim
        conv = dict(cw=lt.conv_w, taps=m.conv_taps, C=self._conv_channels(m), state=pool.tail.get(li)) if m.conv_taps else \
            dict(cw=None, taps=0, C=0, state=None)
        q = torch.empty(meta.T, cq, dtype=torch.float32, device=self.device)
        ops.conv_head(P, 0, meta, ch0=0, ngroups=m.heads * m.maps, gsize=m.dim, normw=lt.q_norm, eps=eps, rot=m.rot_dims,
                      inv_freq=lt.inv_freq, out_dense=q, **conv, **turn)
        col = cq
        if m.kv_from is None:
            ops.conv_head(P, cq, meta, ch0=cq, ngroups=m.kv_heads * m.maps, gsize=m.dim, normw=lt.k_norm, eps=eps,
                          rot=m.rot_dims, inv_freq=lt.inv_freq, pages=pool.k[li], **conv, **turn)
            # values: their own projection, or the key projections once more as they came (no norm, no rotation)
            cv = cq if m.v_from_k else cq + ck
            ops.conv_head(P, cv, meta, ch0=cv, ngroups=m.kv_heads, gsize=m.vdim, normw=None, eps=eps, rot=0,
                          inv_freq=None, pages=pool.v[li], **conv)
            col = cq + ck + (0 if m.v_from_k else m.kv_heads * m.vdim)
        if m.conv_taps > 1:
            ops.conv_state(P, 0, pool.tail[li], m.conv_taps, conv["C"], meta)
        src = self._kv_run[li]
        return ops.paged_attn(q, pool.k[src], pool.v[src], meta, maps=m.maps, H=m.heads, G=m.kv_heads, d=m.dim, vd=m.vdim,
                              window=m.window, keep_first=m.keep_first, scale=m.scale, lam=m.lam, out_scale=m.out_scale,
                              out_norm=m.out_norm, eps=eps, gate=P if m.gate else None, gate0=col, sink=m.sink,
                              chunk=m.chunk, softcap=m.softcap, gate_wide=m.gate and m.gate_channels,
                              sinks=lt.sinks if m.head_sinks else None, slopes=lt.slopes if m.dist_slopes is not None else None)

    def _latent(self, li, m: LatentAttention, lt: LayerTensors, P, meta):
        """Scores of head h are q_h . [W_uk,h c | rotated part] = [W_uk,h^T q_h | rotated query part] . [c | rotated part]:
        the queries are carried into the latent space (one batched product), the kernel attends over the cached rows with
        one key/value head, and W_uv,h is applied to the weighted sum of latent rows afterwards."""
        ops, pool, eps = self.ops, self.pool, self.cfg.norm_eps
        T, H, hd = meta.T, m.heads, m.dim + m.rot_dim
        qd = torch.empty(T, H * hd, dtype=torch.float32, device=self.device)
        no_conv = dict(cw=None, taps=0, C=0, ch0=0, state=None)
        ops.conv_head(P, 0, meta, ngroups=H, gsize=hd, normw=None, eps=eps, rot=m.rot_dims, rot0=m.dim, interleaved=True,
                      inv_freq=lt.inv_freq, out_dense=qd, **no_conv)
        ops.conv_head(P, H * hd, meta, ngroups=1, gsize=m.rank + m.rot_dim, normw=lt.k_norm, norm_n=m.rank, eps=eps,
                      rot=m.rot_dims, rot0=m.rank, interleaved=True, inv_freq=lt.inv_freq, pages=pool.k[li], **no_conv)
        q3 = qd.view(T, H, hd)
        q = torch.empty(T, H, m.rank + m.rot_dim, dtype=torch.float32, device=self.device)
        q[:, :, :m.rank] = torch.bmm(q3[:, :, :m.dim].to(self.act).transpose(0, 1), lt.w_uk).transpose(0, 1)
        q[:, :, m.rank:] = q3[:, :, m.dim:]
        o = ops.paged_attn(q.view(T, -1), pool.k[li], pool.k[li], meta, maps=1, H=H, G=1, d=m.rank + m.rot_dim, vd=m.rank,
                           window=m.window, keep_first=0, scale=m.scale, lam=0.0, out_scale=1.0, out_norm=False, eps=eps)
        o = o.view(T, H, m.rank).transpose(0, 1)
        if not m.gate and m.out_scale == 1.0:
            return torch.bmm(o, lt.w_uv.transpose(1, 2)).transpose(0, 1).reshape(T, H * m.vdim)
        # gated: the head outputs stay float up to the gate, which rounds them once
        if o.dtype == torch.float32 or o.device.type != "cuda":
            of = torch.bmm(o.float(), lt.w_uv.float().transpose(1, 2))
        else:
            of = torch.bmm(o, lt.w_uv.transpose(1, 2), out_dtype=torch.float32)
        of = of.transpose(0, 1).reshape(T, H * m.vdim)
        if not m.gate:
            return (of * m.out_scale).to(self.act)
        return ops.gate_cols(of, P, H * hd + m.rank + m.rot_dim, self.act, m.out_scale)

    def _delta(self, li, m: DeltaRule, lt: LayerTensors, P, meta):
        ops = self.ops
        hd = m.heads * m.dim
        # columns of P: r | k | v | output gate | removal logits | low-rank decay input
        lo = ops.act_cols(P, 5 * hd, m.decay_rank, "tanh")
        arrays = ops.delta_gates(P, 0, hd, 4 * hd, self._linear_f32(lo, lt.w_decay), lt.decay_bias, lt.remove_bias, m.decay_rate,
                                 m.unit_eps, m.heads, m.dim)
        o = ops.delta_scan(arrays, P, 2 * hd, self.pool.matrix[li], m.heads, m.dim, m.dim, meta)
        return ops.head_norm_gate(o, lt.o_norm, P, 3 * hd, m.heads, m.dim, self.cfg.norm_eps, self.act, scale=m.out_scale)

    def _side_by_side(self, li, m: SideBySide, lt: LayerTensors, P, meta):
        nl = lt.left.w_in.shape[0]                   # the left mixer's rows of the stacked projection
        return torch.cat([self._mixer(li, m.left, lt.left, P[:, :nl], meta), self._mixer(li, m.right, lt.right, P[:, nl:], meta)], 1)

    def _mlstm(self, li, m: Mlstm, lt: LayerTensors, P, meta):
        ops, pool = self.ops, self.pool
        hd, hv = m.heads * m.dim, m.heads * m.vdim
        # columns of P: q | k | v | output gate | input gates | forget gates
        a, b, em = ops.mlstm_gates(P, 2 * hd + 2 * hv, lt.gate_bias, m.gate_cap, m.m_start, m.heads, pool.vector[li], meta)
        qf, ff, gf = ops.mlstm_expand(P, 0, hd, a, b, m.heads, m.dim)
        # the normaliser n rides along as one more column of the matrix memory (its value is the constant 1)
        o = ops.hgrn2_scan(qf, ff, P, 2 * hd, pool.matrix[li], m.heads, m.dim, m.vdim + 1, meta, gf=gf, ones_col=True)
        return ops.head_norm_gate(o, lt.o_norm, P, 2 * hd + hv, m.heads, m.vdim, self.cfg.norm_eps, self.act, em=em,
                                  den_floor=m.den_floor)

    # rows per expert (on average) from which the experts run as dense products over their sorted rows; below, every
    # (row, chosen expert) pair is served by the row-wise kernels, which read no more than the chosen experts' weights
    moe_dense_rows = 16

    def _experts(self, f: RoutedExperts, lt: LayerTensors, xa, meta):
        ops = self.ops
        gated = f.act == "swiglu"
        idx, wts = ops.moe_route(xa, lt.w_router, f.groups, f.keep, f.top, f.scale, f.score, f.group_top, f.renorm)
        base = None
        if f.shared_ff:
            a = F.linear(xa, lt.w_sup)
            base = F.linear(ops.glu_pairs(a) if gated else ops.relu2(a), lt.w_sdn)
        if meta.T * f.top < self.moe_dense_rows * f.experts:
            return ops.moe_rows(xa, idx, wts, lt.w_up, lt.w_dn, base, gated)
        y = ops.moe_sorted(xa, idx, wts, lt.w_up, lt.w_dn, base, gated)         # bfloat16: one grouped product per projection
        if y is not None:
            return y
        # rows sorted by expert: one gather, two library products per expert on its run of rows, one weighted sum per row
        T, top = meta.T, f.top
        order = idx.view(-1).sort(stable=True)
        counts = torch.bincount(order.values, minlength=f.experts).tolist()     # (the host learns the runs' lengths)
        pair = order.indices                                                    # pair t * top + j at every sorted place
        xs = xa[pair // top]
        A = torch.empty(T * top, lt.w_up.shape[1], dtype=self.act, device=self.device)
        at = 0
        for e, c in enumerate(counts):
            if c:
                torch.mm(xs[at:at + c], lt.w_up[e].t(), out=A[at:at + c])
                at += c
        A = ops.glu_pairs(A) if gated else ops.relu2(A)
        ys = torch.empty(T * top, self.cfg.width, dtype=self.act, device=self.device)
        at = 0
        for e, c in enumerate(counts):
            if c:
                torch.mm(A[at:at + c], lt.w_dn[e].t(), out=ys[at:at + c])
                at += c
        place = torch.empty_like(pair)
        place[pair] = torch.arange(T * top, device=self.device)
        return ops.moe_combine(ys, place.view(T, top).to(torch.int32), wts, base)

    def _hgrn2(self, li, m: Hgrn2, lt: LayerTensors, P, meta):
        ops = self.ops
        hd = m.heads * m.dim
        qf, ff = ops.hgrn2_gates(P, 0, hd, lt.f_bias, lt.lower, hd)
        o = ops.hgrn2_scan(qf, ff, P, 2 * hd, self.pool.matrix[li], m.heads, m.dim, m.vdim, meta)
        return ops.row_norm(o.view(meta.T * m.heads, m.vdim), lt.o_norm, self.cfg.norm_eps, self.act).view(meta.T, -1)

    # ------------------------------------------------------------------ one step
    @torch.no_grad()
    def step(self, entries: Sequence[tuple], want: Optional[Sequence[Sequence[int]]] = None, collect: Optional[list] = None):
        """``entries``: [(slot, token ids)] with slots from ``pool.admit()``; every entry continues its sequence by
        these tokens.  ``want[i]``: indices into entry i's tokens whose logits are returned (default: the last one).
        Returns float32 logits [wanted rows, vocab] in the order of entries and indices."""
        pool = self.pool
        pairs = self.cfg.pair_embed
        seqs, ids, prs = [], [], []
        for slot, toks in entries:
            if len(toks) == 0:
                raise ValueError("an entry without tokens")
            seqs.append((slot, pool.len_of[slot], len(toks), list(pool.reserve(slot, len(toks)))))
            ids += list(toks)
            if pairs is not None:                    # the previous token is part of the sequence's state
                prs += pairs.rows(pool.last_token[slot], toks)
        rows, at = [], 0
        for b, (_, _, n, _) in enumerate(seqs):
            idx = [n - 1] if want is None else want[b]
            if any(not 0 <= i < n for i in idx):
                raise ValueError("a wanted index outside its entry")
            rows += [at + i for i in idx]
            at += n
        idt = torch.tensor(ids if pairs is None else [ids, prs], dtype=torch.int64)      # [T], or [2, T] with pair rows
        if self.use_graph and collect is None and len(ids) == len(seqs) and rows == list(range(len(seqs))):
            logits = self._decode_step(seqs, idt)
        else:
            if self.device.type == "cuda":
                idt = idt.pin_memory().to(self.device, non_blocking=True)
            logits = self._forward(R.BatchMeta(seqs, self.device), idt, rows, collect)
        for (slot, _, n, _), (_, toks) in zip(seqs, entries):
            pool.commit(slot, n, last_token=int(toks[-1]))
        return logits

    def _decode_step(self, seqs, idt):
        """One token per sequence.  The first step of a shape runs kernel by kernel (and loads whatever is loaded
        lazily); the second is recorded -- recording executes nothing, so cache and state are touched once per step --
        and from then on a step is: refill the static batch description and token ids, replay."""
        B = len(seqs)
        width = 1
        while width < max(len(pg) for *_, pg in seqs):
            width *= 2
        ent = self._graphs.get((B, width))
        if ent is None:
            self._graphs[(B, width)] = {}
            return self._forward(R.BatchMeta(seqs, self.device), idt.pin_memory().to(self.device, non_blocking=True),
                                 list(range(B)), None)
        if not ent:
            ent["meta"] = R.BatchMeta(seqs, self.device, max_pages=width, static=True)
            ent["host_ids"] = torch.empty(idt.shape, dtype=torch.int64, pin_memory=True)
            ent["ids"] = torch.zeros(idt.shape, dtype=torch.int64, device=self.device)
            self.ops.before_recording(ent["meta"])       # whatever the operations would otherwise build on first use
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                ent["logits"] = self._forward(ent["meta"], ent["ids"], list(range(B)), None)
            ent["graph"] = graph
        if "done" in ent:
            ent["done"].synchronize()                    # the last replay has read the pinned buffers refilled below
        ent["meta"].update(seqs)
        ent["host_ids"].copy_(idt)
        ent["ids"].copy_(ent["host_ids"], non_blocking=True)
        ent["graph"].replay()
        ent.setdefault("done", torch.cuda.Event()).record()
        self.graph_replays += 1
        return ent["logits"].clone()

    def _mixer(self, li, m, lt, P, meta):
        if isinstance(m, WindowAttention):
            return self._attention(li, m, lt, P, meta)
        if isinstance(m, LatentAttention):
            return self._latent(li, m, lt, P, meta)
        if isinstance(m, Mlstm):
            return self._mlstm(li, m, lt, P, meta)
        if isinstance(m, DeltaRule):
            return self._delta(li, m, lt, P, meta)
        if isinstance(m, SideBySide):
            return self._side_by_side(li, m, lt, P, meta)
        return self._hgrn2(li, m, lt, P, meta)

    def _forward(self, meta, idt, rows, collect):
        cfg, ops = self.cfg, self.ops
        if cfg.pair_embed is not None:
            x = ops.embed_rows(idt[0], self.embed, idt[1], self.pair_table, cfg.embed_scale)
        else:
            x = ops.embed_rows(idt, self.embed, scale=cfg.embed_scale)
        if cfg.block == "sandwich":
            self._sandwich_layers(x, meta, collect)
        elif cfg.block == "parallel":
            x = self._parallel_layers(x, meta, collect)
        elif cfg.block == "pre_norm":
            x = self._prenorm_layers(x, meta, collect)
        else:
            xa = x.to(self.act)
            for ri, li in enumerate(self.runs):
                m, mlp, lt = cfg.mixers[li], cfg.mlps[li], self.layers[li]
                a = self._mixer(ri, m, lt, F.linear(xa, lt.w_in, lt.b_in), meta)
                xa = ops.sum_group_norm(x, F.linear(a, lt.w_out), lt.norm1, cfg.norm_groups, cfg.residual_alpha, cfg.norm_eps,
                                        self.act)
                if mlp is not None:
                    a = ops.clamped_glu(F.linear(xa, lt.w_gu), mlp.limit, mlp.slope)
                    xa = ops.sum_group_norm(x, F.linear(a, lt.w_down), lt.norm2, cfg.norm_groups, cfg.residual_alpha,
                                            cfg.norm_eps, self.act)
                if collect is not None:
                    collect.append(x.clone())
        if not rows:
            return torch.empty(0, cfg.vocab, dtype=torch.float32, device=self.device)
        if rows == list(range(meta.T)):
            xr = x                                # (the final norm writes its own output)
        else:
            xr = x[torch.tensor(rows, dtype=torch.int64, device=self.device)].contiguous()
        xo = torch.empty_like(xr)
        xa = ops.sum_group_norm(xr, None, self.final_norm, cfg.norm_groups, 1.0, cfg.norm_eps, self.act, x_out=xo)
        logits = F.linear(xa, self.head).float()
        if cfg.logit_softcap > 0:
            logits = torch.tanh(logits / cfg.logit_softcap) * cfg.logit_softcap
        return logits

    def _sandwich_layers(self, x, meta, collect):
        """x <- x + norm_b(f(norm_a(x))) for the mixer and the feed-forward of every layer; x float32, in place.  The norm
        behind a sublayer, the residual sum and the norm in front of the next sublayer are one kernel."""
        cfg, ops, eps = self.cfg, self.ops, self.cfg.norm_eps
        n = len(self.runs)
        xa = ops.row_norm(x, self.layers[self.runs[0]].norm1, eps, self.act) if n else None
        for ri, li in enumerate(self.runs):
            m, mlp, lt = cfg.mixers[li], cfg.mlps[li], self.layers[li]
            nxt = self.layers[self.runs[ri + 1]].norm1 if ri + 1 < n else None
            a = self._mixer(ri, m, lt, F.linear(xa, lt.w_in, lt.b_in), meta)
            xa = ops.post_norm_add(x, F.linear(a, lt.w_out), lt.norm1b, nxt if mlp is None else lt.norm2, eps, self.act)
            if isinstance(mlp, RoutedExperts):
                xa = ops.post_norm_add(x, self._experts(mlp, lt, xa, meta), lt.norm2b, nxt, eps, self.act)
            elif mlp is not None:
                raise ValueError("the sandwich form has no such feed-forward yet")
            if collect is not None:
                collect.append(x.clone())

    def _parallel_layers(self, x, meta, collect):
        """u = norm(x), x <- x + mixer(u) + ff(u): both sublayers read one normed copy of the stream, their outputs join it
        in one kernel that also norms the stream for the next execution.  In front of the executions of ``cfg.mix_in``
        the stream becomes W_mix [x ; e], e the embedding output (bfloat16 operands, 32-bit result)."""
        cfg, ops, eps = self.cfg, self.ops, self.cfg.norm_eps
        mix_in = set(cfg.mix_in)
        e_act = x.to(self.act, copy=True) if mix_in else None      # (the stream itself is updated in place below)
        n, xa = len(self.runs), None
        for ri, li in enumerate(self.runs):
            m, mlp, lt = cfg.mixers[li], cfg.mlps[li], self.layers[li]
            if ri in mix_in:
                x = self._linear_f32(torch.cat([x.to(self.act), e_act], 1), self.w_mix)
                xa = None
            if xa is None:
                xa = ops.add_norm(x, None, None, lt.norm1, eps, self.act)
            P = F.linear(xa, lt.w_in, lt.b_in)       # [mixer's projections | up projection of a dense feed-forward]
            y1 = F.linear(self._mixer(ri, m, lt, P, meta), lt.w_out)
            if isinstance(mlp, DenseMlp):
                y2 = F.linear(ops.act_cols(P, P.shape[1] - mlp.ff, mlp.ff, mlp.act), lt.w_down, lt.b_down)
            elif isinstance(mlp, RoutedExperts):
                y2 = self._experts(mlp, lt, xa, meta)
            elif mlp is None:
                y2 = None
            else:
                raise ValueError("the parallel block has no such feed-forward")
            nxt = self.layers[self.runs[ri + 1]].norm1 if ri + 1 < n and ri + 1 not in mix_in else None
            xa = ops.add_norm(x, y1, y2, nxt, eps, self.act)
            if collect is not None:
                collect.append(x.clone())
        return x

    def _prenorm_layers(self, x, meta, collect):
        """x <- x + f(norm(x)) for the mixer and then the feed-forward of every execution, on a stream of ``cfg.streams``
        copies X[s] (all equal to the embedding output at first): sublayer f reads u = sum_s in[s] X[s] and writes
        X[t] <- sum_s mix[s, t] X[s] + out[t] f(norm(u)).  The write-back of one sublayer, the read-out of the next and its
        norm are one kernel.  Returns the sum of the copies."""
        cfg, ops, eps = self.cfg, self.ops, self.cfg.norm_eps
        S = cfg.streams
        X = x[:, None, :].repeat(1, S, 1)
        y = prev = None
        for ri, li in enumerate(self.runs):
            m, mlp, lt = cfg.mixers[li], cfg.mlps[li], self.layers[li]
            xa, _ = ops.hc_step(X, y, prev, lt.hc1, lt.norm1, eps, self.act)
            y, prev = F.linear(self._mixer(ri, m, lt, F.linear(xa, lt.w_in, lt.b_in), meta), lt.w_out), lt.hc1
            if isinstance(mlp, DenseMlp):
                if mlp.bias:
                    raise ValueError("the sequential pre-norm block's dense feed-forward has no biases")
                xa, _ = ops.hc_step(X, y, prev, lt.hc2, lt.norm2, eps, self.act)
                a = F.linear(xa, lt.w_ff)
                y, prev = F.linear(ops.act_cols(a, 0, mlp.ff, mlp.act, lt.act_params or (0.0, 0.0)), lt.w_down, lt.b_down), lt.hc2
            elif mlp is not None:
                raise ValueError("the sequential pre-norm block has no such feed-forward yet")
            if collect is not None:
                ops.hc_step(X, y, prev, None, None, eps, self.act)
                y = prev = None
                collect.append(X.sum(1))
        return ops.hc_step(X, y, prev, self._sum_read, None, eps, self.act, want_u=True)[1]

    def _linear_f32(self, a, w):
        """a w^T with the operands in the activation type and a float32 result (no rounding of the 32-bit accumulator)"""
        if a.dtype == torch.float32 or a.device.type != "cuda":
            return F.linear(a.float(), w.float())
        return torch.mm(a, w.t(), out_dtype=torch.float32)

    # ------------------------------------------------------------------ generation
    @torch.no_grad()
    def generate(self, input_ids, max_new_tokens: int = 32, do_sample=False, temperature=1.0, top_k=0, top_p=1.0,
                 eos_token_id=None, streamer=None, max_prefill_tokens: int = 4096, **_):
        """Greedy / sampling generation for a [B, S] batch of equally long prompts (rows are independent sequences),
        through the same scheduler that serves requests."""
        from ..serving.continuous import generate_batch
        ids = torch.as_tensor(input_ids)
        prompts = [row.tolist() for row in ids.view(-1, ids.shape[-1])]
        t0 = time.perf_counter()
        outs = generate_batch(self, prompts, max_new_tokens=max_new_tokens, max_num_seqs=len(prompts),
                              eos_token_id=eos_token_id, do_sample=do_sample, temperature=temperature, top_k=top_k, top_p=top_p)
        dt = time.perf_counter() - t0
        self.rest_cost_mean = dt / max(1, max_new_tokens)
        width = max(len(o) for o in outs)
        pad = eos_token_id if isinstance(eos_token_id, int) else 0
        gen = torch.tensor([o + [pad] * (width - len(o)) for o in outs], dtype=torch.int64)
        out = torch.cat([ids.view(-1, ids.shape[-1]).cpu(), gen], 1)
        if streamer is not None:
            streamer.put(ids.cpu())
            streamer.put(gen)
            streamer.end()
        return out

    def weight_bytes(self):
        ts = [self.embed, self.head, self.final_norm] + [t for t in (self.pair_table, self.w_mix) if t is not None]
        for lt in self.layers:
            ts += [t for t in vars(lt).values() if isinstance(t, torch.Tensor)]
        return sum(t.numel() * t.element_size() for t in ts)
