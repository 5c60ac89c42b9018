"""A plain, slow implementation of Qwen2-MoE for whole sequences: no cache, no batching, one function per
part, written from the reference's formulas.  It shares no code with the package under test: it reads
config.json and model.safetensors through the ``safetensors`` and ``json`` libraries and computes with
plain torch operations on the CPU, by default in float64.

Every function cites the lines of the reference it follows.  Where the reference has no formula for an
option of this architecture (``norm_topk_prob`` false, a window on Qwen layers, which layers are sparse),
the choice is spelled out in the function.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np
import torch


# ----------------------------------------------------------------------------- basic operations
def matvec_rows(w: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """y[..., i] = sum_j w[i, j] * x[..., j]: weights are row-major [out, in]
    (/root/reference/src/engine/tq_ops.c:287-291)."""
    return torch.einsum("ij,...j->...i", w, x)


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """ss = sum(x^2) / n + eps; out = x * (1 / sqrt(ss)) * weight
    (/root/reference/src/engine/tq_ops.c:1402-1409)."""
    ss = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1] + eps
    return x * (1.0 / torch.sqrt(ss)) * weight


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x)) (/root/reference/src/engine/tq_ops.c:1473-1476)."""
    return x / (1.0 + torch.exp(-x))


def softmax(x: torch.Tensor) -> torch.Tensor:
    """exp(x - max) / sum over the last dimension (/root/reference/src/engine/tq_ops.c:1496-1519)."""
    e = torch.exp(x - x.max(dim=-1, keepdim=True).values)
    return e / e.sum(dim=-1, keepdim=True)


def rope_frequencies(rotary_dim: int, theta: float) -> np.ndarray:
    """freq_i = 1 / powf(base, 2 i / dim), evaluated in float32 like the reference
    (/root/reference/src/engine/tq_ops.c:1424)."""
    out = np.empty(rotary_dim // 2, dtype=np.float32)
    for i in range(rotary_dim // 2):
        expo = np.float32(np.float32(2.0) * np.float32(i) / np.float32(rotary_dim))
        out[i] = np.float32(1.0) / np.power(np.float32(theta), expo, dtype=np.float32)
    return out


def rope(x: torch.Tensor, positions, theta: float, pairing: str = "half", rotary_dim: int | None = None) -> torch.Tensor:
    """Rotates x [T, heads, head_dim] by the angle pos * freq_i (a float32 product,
    /root/reference/src/engine/tq_ops.c:1425) on pair i:
    "interleaved" pairs (x[2i], x[2i+1]) (tq_ops.c:1428-1431);
    "half" pairs (x[i], x[i + dim/2]) (/root/reference/src/engine/tq_transformer.c:1263-1289).
    (a, b) <- (a cos - b sin, a sin + b cos)."""
    T, nh, hd = x.shape
    rot = hd if rotary_dim is None else rotary_dim
    freqs = rope_frequencies(rot, theta)
    pos = np.asarray(positions, dtype=np.float32)
    theta_pi = (pos[:, None] * freqs[None, :]).astype(np.float32)      # float32 product, as in the reference
    ang = torch.from_numpy(theta_pi.astype(np.float64)).to(x.dtype)
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    half = rot // 2
    if pairing == "interleaved":
        a, b = x[..., 0:rot:2], x[..., 1:rot:2]
        out[..., 0:rot:2] = a * cos - b * sin
        out[..., 1:rot:2] = a * sin + b * cos
    elif pairing == "half":
        a, b = x[..., :half], x[..., half:rot]
        out[..., :half] = a * cos - b * sin
        out[..., half:rot] = a * sin + b * cos
    else:
        raise ValueError(pairing)
    return out


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int | None = None,
              scale: float | None = None) -> torch.Tensor:
    """q [T, nh, hd], k and v [T, nkv, hd] of one sequence at positions 0..T-1.
    For the token at position p and head h: kv head h / (nh / nkv)
    (/root/reference/src/engine/tq_transformer.c:1675-1679); scores of positions start..p,
    start = p + 1 - window if p + 1 > window else 0 (:1646-1654), each (q . k) / sqrt(hd) (:1908-1937);
    softmax (:1960); output = sum of p_t v_t (:1975-1976)."""
    T, nh, hd = q.shape
    nkv = k.shape[1]
    sc = 1.0 / math.sqrt(hd) if scale is None else scale
    out = torch.zeros_like(q)
    for p in range(T):
        seq_len = p + 1
        start = seq_len - window if (window is not None and seq_len > window) else 0
        for h in range(nh):
            kvh = h // (nh // nkv)
            s = (k[start:seq_len, kvh, :] @ q[p, h, :]) * sc
            pr = softmax(s)
            out[p, h, :] = pr @ v[start:seq_len, kvh, :]
    return out


def route(x: torch.Tensor, router: torch.Tensor, top_k: int, renormalize: bool, other_side=None):
    """x [H].  logits = router x; top-k by k passes of a scan with >=, so among equals the highest index
    wins and ids come out by descending logit (/root/reference/src/engine/tq_moe.c:611-645).
    renormalize true: softmax over the selected logits (tq_moe.c:648-678).
    renormalize false (no formula in the reference, which always renormalises): softmax over all experts,
    the selected probabilities kept as they are.
    ``other_side`` = (i, j): the choice that an arithmetic with other rounding makes when the expert of rank i (one
    of the chosen, 0 the best) and the expert of rank j (one of those left out) nearly tie: the latter takes the
    former's place."""
    logits = matvec_rows(router, x)
    E = logits.shape[0]
    used, ids = [False] * E, []
    for _ in range(top_k if other_side is None else other_side[1] + 1):
        best, best_val = -1, -math.inf
        for e in range(E):
            if not used[e] and logits[e].item() >= best_val:
                best_val, best = logits[e].item(), e
        used[best] = True
        ids.append(best)
    if other_side is not None:
        i, j = other_side
        ids = ids[:i] + [ids[j]] + ids[i + 1:top_k]
    sel = logits[ids]
    if renormalize:
        w = softmax(sel)
    else:
        w = softmax(logits)[ids]
    return ids, w


def route_margin(x: torch.Tensor, router: torch.Tensor, top_k: int) -> float:
    """How far the last selected logit lies above the best one left out, in units of the logits' spread:
    a small margin means that a rounding error upstream can change which experts run."""
    logits = matvec_rows(router, x)
    if top_k >= logits.shape[0]:
        return math.inf
    top = torch.sort(logits, descending=True).values
    return float((top[top_k - 1] - top[top_k]) / (logits.std() + 1e-30))


def swiglu_mlp(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """down (silu(gate x) * (up x)) (/root/reference/src/engine/tq_transformer.c:2770-2806; experts:
    /root/reference/src/engine/tq_moe.c:864-999 with an exact exponential)."""
    return matvec_rows(down, silu(matvec_rows(gate, x)) * matvec_rows(up, x))


def near_swaps(x: torch.Tensor, router: torch.Tensor, top_k: int, reach: int = 3, spread: float | None = None) -> list:
    """(gap, i, j) for every chosen rank i and every rank j among the ``reach`` best left out, the gap being the
    difference of their logits in units of the logits' spread (the token's own, unless one is given), smallest
    first."""
    logits = matvec_rows(router, x)
    top = torch.sort(logits, descending=True).values
    spread = (float(logits.std()) if spread is None else spread) + 1e-30
    out = [(float(top[i] - top[j]) / spread, i, j) for i in range(top_k) for j in range(top_k, min(top_k + reach, len(top)))]
    return sorted(out)


def moe(x: torch.Tensor, w: dict, top_k: int, renormalize: bool, margins: list | None = None,
        other_side=None, swaps: list | None = None) -> torch.Tensor:
    """x [T, H].  out = sum over the selected experts, in the order selected, of weight * expert(x)
    (/root/reference/src/engine/tq_moe.c:720,864-999); then + sigmoid(x . shared_scale) * shared(x)
    (tq_moe.c:1005-1058)."""
    out = torch.zeros_like(x)
    # with two experts a token's own spread is the gap itself: there the unit is the spread over all the step's tokens
    spread = None
    if swaps is not None and w["router"].shape[0] == 2 and x.shape[0] > 1:
        spread = float(torch.stack([matvec_rows(w["router"], x[t]) for t in range(x.shape[0])]).std())
    for t in range(x.shape[0]):
        ids, wts = route(x[t], w["router"], top_k, renormalize, other_side=(other_side or {}).get(t))
        if swaps is not None:
            swaps.append(near_swaps(x[t], w["router"], top_k, spread=spread))
        if margins is not None:
            margins.append(route_margin(x[t], w["router"], top_k))
        acc = torch.zeros_like(x[t])
        for e, wt in zip(ids, wts):
            acc = acc + wt * swiglu_mlp(x[t], w["experts"][e]["gate"], w["experts"][e]["up"], w["experts"][e]["down"])
        if "shared" in w:
            g = 1.0
            if "shared_scale" in w:
                g = 1.0 / (1.0 + torch.exp(-(x[t] @ w["shared_scale"].reshape(-1))))
            acc = acc + g * swiglu_mlp(x[t], w["shared"]["gate"], w["shared"]["up"], w["shared"]["down"])
        out[t] = acc
    return out


# ----------------------------------------------------------------------------- the model
class PlainQwen2Moe:
    """Reads a model folder and computes the logits of whole sequences."""

    def __init__(self, model_dir: str, dtype: torch.dtype = torch.float64, rope_pairing: str = "half"):
        from safetensors import safe_open
        with open(os.path.join(model_dir, "config.json")) as f:
            self.cfg = json.load(f)
        self.dtype = dtype
        self.rope_pairing = rope_pairing
        self.t = {}
        with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
            for name in f.keys():
                self.t[name] = f.get_tensor(name).to(dtype)
        c = self.cfg
        self.L, self.H = c["num_hidden_layers"], c["hidden_size"]
        self.nh = c["num_attention_heads"]
        self.nkv = c.get("num_key_value_heads", self.nh)
        self.hd = c.get("head_dim") or self.H // self.nh
        self.eps = c["rms_norm_eps"]
        # the rotation's base: a key of its own, or inside the object that newer folders write
        self.theta = c["rope_theta"] if c.get("rope_theta") is not None else c["rope_parameters"]["rope_theta"]
        self.has_bias = c.get("qkv_bias", True)
        self.margins: dict[int, list] = {}      # per sparse layer, the routing margin of every token of the last call
        self.swaps: dict[int, list] = {}        # per sparse layer and token, the nearest exchanges of two experts
        self.other_side: dict = {}              # (layer, position) -> (i, j): near-ties that calls decide the other way

    def layer_is_sparse(self, l: int) -> bool:
        """No rule in the reference (it looks for a router tensor, /root/reference/src/engine/tq_model.c:3440-3444);
        the configuration's rule: not in mlp_only_layers, experts exist, (l + 1) % decoder_sparse_step == 0."""
        c = self.cfg
        return (l not in c.get("mlp_only_layers", []) and c["num_experts"] > 0
                and (l + 1) % c.get("decoder_sparse_step", 1) == 0)

    def layer_window(self, l: int):
        """Layers from max_window_layers on see the last sliding_window positions when use_sliding_window is set
        (window arithmetic of /root/reference/src/engine/tq_transformer.c:1646-1654, which the reference applies
        to another model family only)."""
        c = self.cfg
        if c.get("layer_types") is not None:      # a folder that lists its layers' kinds is taken at its word
            return c["sliding_window"] if c["layer_types"][l] == "sliding_attention" else None
        if c.get("use_sliding_window", False) and l >= c.get("max_window_layers", self.L):
            return c["sliding_window"]
        return None

    def attention_layer(self, l: int, xb: torch.Tensor) -> torch.Tensor:
        """q, k, v with bias right after the product (/root/reference/src/engine/tq_transformer.c:1040-1093),
        rotation of q and k (:1342-1344), attention, output projection (:2239-2240)."""
        p, t = f"model.layers.{l}.self_attn.", self.t
        T = xb.shape[0]
        q, k, v = (matvec_rows(t[p + n + "_proj.weight"], xb) for n in "qkv")
        if self.has_bias:
            q, k, v = q + t[p + "q_proj.bias"], k + t[p + "k_proj.bias"], v + t[p + "v_proj.bias"]
        q, k, v = q.view(T, self.nh, self.hd), k.view(T, self.nkv, self.hd), v.view(T, self.nkv, self.hd)
        pos = list(range(T))
        q, k = rope(q, pos, self.theta, self.rope_pairing), rope(k, pos, self.theta, self.rope_pairing)
        o = attention(q, k, v, window=self.layer_window(l))
        return matvec_rows(t[p + "o_proj.weight"], o.reshape(T, self.nh * self.hd))

    def ffn_layer(self, l: int, xb: torch.Tensor) -> torch.Tensor:
        p, t, c = f"model.layers.{l}.mlp.", self.t, self.cfg
        if not self.layer_is_sparse(l):
            return swiglu_mlp(xb, t[p + "gate_proj.weight"], t[p + "up_proj.weight"], t[p + "down_proj.weight"])
        w = {"router": t[p + "gate.weight"],
             "experts": [{n: t[f"{p}experts.{e}.{n}_proj.weight"] for n in ("gate", "up", "down")}
                         for e in range(c["num_experts"])]}
        if c["shared_expert_intermediate_size"] > 0:
            w["shared"] = {n: t[f"{p}shared_expert.{n}_proj.weight"] for n in ("gate", "up", "down")}
            w["shared_scale"] = t[p + "shared_expert_gate.weight"]
        self.margins[l], self.swaps[l] = [], []
        return moe(xb, w, c["num_experts_per_tok"], c.get("norm_topk_prob", False), self.margins[l],
                   other_side={pos: ij for (layer, pos), ij in self.other_side.items() if layer == l}, swaps=self.swaps[l])

    def logits(self, tokens) -> torch.Tensor:
        """Logits [T, vocab] at every position of one sequence (step order of
        /root/reference/src/engine/tq_transformer.c:2281-3029)."""
        t = self.t
        x = t["model.embed_tokens.weight"][list(tokens)]                       # no scaling (:2297-2329)
        for l in range(self.L):
            xb = rmsnorm(x, t[f"model.layers.{l}.input_layernorm.weight"], self.eps)        # :2494
            x = x + self.attention_layer(l, xb)                                               # :2268
            xb = rmsnorm(x, t[f"model.layers.{l}.post_attention_layernorm.weight"], self.eps)  # :2685, :2722
            x = x + self.ffn_layer(l, xb)                                                     # :2701, :2823
        x = rmsnorm(x, t["model.norm.weight"], self.eps)                                      # :2922
        head = t["lm_head.weight"] if "lm_head.weight" in t else t["model.embed_tokens.weight"]   # tq_model.c:1499-1516
        return matvec_rows(head, x)                                                           # :2931-2942

    def near_ties(self, bound: float, position: int | None = None) -> list:
        """(gap, layer, position, i, j) of every exchange of a chosen expert (rank i) for one left out (rank j) in
        the last ``logits`` call whose gap is under ``bound``, at ``position`` or at all positions, smallest first."""
        out = []
        for l in sorted(self.swaps):
            for p in (range(len(self.swaps[l])) if position is None else [position]):
                out += [(gap, l, p, i, j) for gap, i, j in self.swaps[l][p] if gap < bound]
        return sorted(out)

    def min_margins(self) -> torch.Tensor:
        """For every token of the last ``logits`` call, its smallest routing margin over the sparse layers."""
        if not self.margins:
            return torch.empty(0)
        return torch.tensor([self.margins[l] for l in sorted(self.margins)]).min(dim=0).values


# ----------------------------------------------------------------------------- sampling and generation
def sample_argmax(logits) -> int:
    """First maximum wins (/root/reference/src/engine/tq_generate.c:30-40)."""
    best, best_val = 0, logits[0]
    for i in range(1, len(logits)):
        if logits[i] > best_val:
            best_val, best = logits[i], i
    return best


class PlainRng:
    """xorshift64* to a float in [0, 1) (/root/reference/src/engine/tq_generate.c:53-58)."""

    def __init__(self, seed: int):
        self.s = seed if seed else 42
        self.s &= (1 << 64) - 1

    def next(self) -> float:
        m = (1 << 64) - 1
        self.s ^= self.s >> 12
        self.s ^= (self.s << 25) & m
        self.s ^= self.s >> 27
        return float(np.float32(((self.s * 0x2545F4914F6CDD1D) & m) >> 33) / np.float32(1 << 31))


def sample_topp(logits: np.ndarray, temperature: float, top_p: float, rng: PlainRng) -> int:
    """/root/reference/src/engine/tq_generate.c:81-156 in float32: greedy if temperature or top_p is not
    positive; keep logits >= max - 16 T; p = exp((l - max) / T) normalised; sort descending (ties: by index,
    the reference's qsort leaves them unspecified); cut where the running sum reaches top_p; r = u * that sum;
    walk until the running sum reaches r."""
    logits = np.asarray(logits, dtype=np.float32)
    if temperature <= 0.0 or top_p <= 0.0:
        return sample_argmax(logits)
    mx = logits.max()
    thr = np.float32(mx - np.float32(16.0) * np.float32(temperature))
    inv_t = np.float32(1.0) / np.float32(temperature)
    idx = np.nonzero(logits >= thr)[0]
    p = np.exp((logits[idx] - mx) * inv_t).astype(np.float32)
    s = np.float32(0.0)
    for v in p:
        s = np.float32(s + v)
    p = (p * (np.float32(1.0) / s)).astype(np.float32)
    order = np.argsort(-p, kind="stable")
    p, idx = p[order], idx[order]
    cum, n_top = np.float32(0.0), 0
    for i in range(len(p)):
        cum = np.float32(cum + p[i])
        n_top = i + 1
        if cum >= np.float32(top_p):
            break
    r = np.float32(np.float32(rng.next()) * cum)
    cdf = np.float32(0.0)
    for i in range(n_top):
        cdf = np.float32(cdf + p[i])
        if cdf >= r:
            return int(idx[i])
    return int(idx[0])


def apply_rep_penalty(logits: np.ndarray, recent: list, window: int, penalty: float) -> None:
    """Over the last min(len, window) tokens, newest first, once per occurrence: a positive logit is divided
    by the penalty, any other multiplied (/root/reference/src/engine/tq_generate.c:387-400)."""
    if penalty <= 1.0:
        return
    n = min(len(recent), window)
    for r in range(n):
        tok = recent[len(recent) - 1 - r]
        if 0 <= tok < len(logits):
            logits[tok] = logits[tok] / np.float32(penalty) if logits[tok] > 0 else logits[tok] * np.float32(penalty)


def generate(model: PlainQwen2Moe, prompt, max_tokens: int, temperature: float = 0.0, top_p: float = 0.9,
             seed: int = 42, rep_penalty: float = 1.0, rep_window: int = 32, stop_tokens=(),
             loop_detection: bool = False) -> list:
    """The reference's loop for one prompt (/root/reference/src/engine/tq_generate.c:363-630): penalty, sample;
    while fewer than max_tokens are out: stop on an end token, emit, run, penalty, sample, and (``loop_detection``)
    stop when the 4-gram that the new token closes has been seen three times before (:611-629; the tokens
    hashed are the prompt's last ``rep_window`` and every sampled one, :381-384, and the first sampled token,
    drawn before the loop, is not looked at, :403-410).  Every step recomputes the whole sequence."""
    rng = PlainRng(seed)
    seq = list(prompt)
    rep_window = min(rep_window, 128)                                     # :367
    recent = list(prompt[-rep_window:]) if rep_window else []
    out, ring, n_hashed = [], [], 0
    while len(out) < max_tokens:
        logits = model.logits(seq)[-1].to(torch.float32).numpy().copy()
        apply_rep_penalty(logits, recent, rep_window, rep_penalty)
        nxt = sample_topp(logits, temperature, top_p, rng)
        recent.append(nxt)
        if loop_detection and len(seq) > len(prompt) and len(recent) >= 4:
            h = 0
            for t in recent[-4:]:
                h = (h * 31 + t) % (1 << 32)
            matches = sum(1 for x in ring if x == h)
            if len(ring) < 64:
                ring.append(h)
            else:
                ring[n_hashed % 64] = h
            n_hashed += 1
            if matches >= 3:
                break
        if nxt in stop_tokens:
            break
        out.append(nxt)
        seq.append(nxt)
    return out
