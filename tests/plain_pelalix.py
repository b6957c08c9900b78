"""The Pelalix design, plain and slow: whole sequences on the CPU in float64, no cache, no batching, one function
per mechanism.  The GPU tests compare the framework with this file; it shares no code with the product."""
import math

import torch

F64 = torch.float64


def dynamic_tanh(x, weight, bias, alpha):
    """y = tanh(alpha x) * weight + bias, element by element."""
    return torch.tanh(alpha * x) * weight + bias


def token_shift(x, mix, before=None):
    """Row t becomes x[t] + (x[t-1] - x[t]) * mix with the ORIGINAL row t-1; the row before the first one is
    `before` (zeros if not given)."""
    first = torch.zeros_like(x[:1]) if before is None else before.reshape(1, -1).to(x.dtype)
    earlier = torch.cat([first, x[:-1]], dim=0)
    return x + (earlier - x) * mix


def rms_norm_whole(x, weight, eps):
    """Every row divided by its root mean square taken over ALL its entries, then times the weight."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def blend_values(v, v_source, lam):
    return (1.0 - lam) * v + lam * v_source


def raw_scores(q, k, scale):
    """q [T, H, d], k [T, G, d] -> [H, T, T]; query head h reads key head h // (H / G)."""
    H, G = q.shape[1], k.shape[1]
    out = torch.empty(H, q.shape[0], k.shape[0], dtype=q.dtype)
    for h in range(H):
        out[h] = q[:, h, :] @ k[:, h // (H // G), :].T * scale
    return out


def mix_heads(scores, talk):
    """scores [H, T, T]; head h gets sum_g talk[h, g] * scores[g]."""
    return torch.einsum("hg,gij->hij", talk, scores)


def softmax_with_sink(scores, sink):
    """Causal softmax over the keys j <= i whose denominator also holds exp(sink_h), once per row; the sink has no
    value, so a row's weights add up to less than one.  `sink` None: the usual softmax."""
    H, T, S = scores.shape
    assert T == S
    allowed = torch.tril(torch.ones(T, T, dtype=torch.bool))
    s = scores.masked_fill(~allowed, -math.inf)
    top = s.amax(dim=-1, keepdim=True)
    if sink is not None:
        top = torch.maximum(top, sink.view(H, 1, 1))
    e = torch.exp(s - top)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink.view(H, 1, 1) - top)
    return e / den


def weighted_values(p, v):
    """p [H, T, T], v [T, G, e] -> [T, H, e]."""
    H, G = p.shape[0], v.shape[1]
    return torch.stack([p[h] @ v[:, h // (H // G), :] for h in range(H)], dim=1)


def head_gate(out, x, w_gate):
    """Every head's result times sigmoid of one number per head, made from the mixer's input."""
    return out * torch.sigmoid(x @ w_gate.T).unsqueeze(-1)


def gated_mlp(x, w_gate, w_up, w_down):
    g = x @ w_gate.T
    return (g * torch.sigmoid(g) * (x @ w_up.T)) @ w_down.T


def attention_mixer(cfg_mixer, w, p, x, eps, v_source):
    """The whole mixer on its (shifted) input x [T, W]; returns (result, the values it used)."""
    T = x.shape[0]
    H, G, d, e = cfg_mixer["heads"], cfg_mixer["kv_heads"], cfg_mixer["dim"], cfg_mixer["vdim"]
    q = rms_norm_whole(x @ w[p + "q"].T, w[p + "q.norm"], eps).view(T, H, d)
    k = rms_norm_whole(x @ w[p + "k"].T, w[p + "k.norm"], eps).view(T, G, d)
    v = (x @ w[p + "v"].T).view(T, G, e)
    if v_source is not None:
        v = blend_values(v, v_source, w[p + "vmix"])
    s = mix_heads(raw_scores(q, k, cfg_mixer["scale"]), w[p + "talk"])
    out = weighted_values(softmax_with_sink(s, w[p + "sink"]), v)
    out = head_gate(out, x, w[p + "g"])
    return out.reshape(T, H * e) @ w[p + "o"].T, v


def forward(cfg, weights, tokens, streams=None):
    """Logits [T, vocab] of the whole sequence.  `streams`, a list, collects the residual stream after every layer."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    h = w["embed"][torch.tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    v_source = None
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = dynamic_tanh(h, w[p + "norm1"], w[p + "norm1.b"], w[p + "norm1.alpha"])
        x = token_shift(x, w[p + "shift"])
        mixes = bool(layer["mixer"].get("v_mix"))
        a, v = attention_mixer(layer["mixer"], w, p + "mix.", x, eps, v_source if mixes else None)
        if mixes and v_source is None:
            v_source = v
        h = h + a * w[p + "ls1"]
        if layer["mlp"] is not None:
            x = dynamic_tanh(h, w[p + "norm2"], w[p + "norm2.b"], w[p + "norm2.alpha"])
            h = h + gated_mlp(x, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"]) * w[p + "ls2"]
        if streams is not None:
            streams.append(h.clone())
    x = dynamic_tanh(h, w["final.norm"], w["final.norm.b"], w["final.norm.alpha"])
    return x @ w["head"].T


def greedy(logits) -> int:
    return int(torch.argmax(logits))
