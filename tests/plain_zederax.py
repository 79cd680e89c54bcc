"""A plain, slow Zederax: whole sequences, no cache, float64 by default. One function per mechanism; nothing here is
shared with the engine. Weights are a dict keyed by the checkpoint tensor names (``embed``, ``l0.mix.q`` ...), the
configuration is the raw ``config.json`` dict.

Notation: T tokens, D the model width, H query heads, G key/value heads, dk the size of a query/key head, dv of a value
head, F the inner width of the feed-forward. i is the position of a query, j of a key.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

Tensor = torch.Tensor


def unit_rms(x: Tensor, eps: float) -> Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    return unit_rms(x, eps) * weight


def head_slopes(n_heads: int, dtype=torch.float64) -> Tensor:
    """Head h (from 0) of H: 2^(-8 (h + 1) / H)."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / n_heads) for h in range(n_heads)], dtype=dtype)


def soft_cap(s: Tensor, cap: Optional[float]) -> Tensor:
    return s if not cap else cap * torch.tanh(s / cap)


def visible(n: int, window: Optional[int]) -> Tensor:
    """[i, j]: True where query i sees key j: j <= i, and with a window i - j < window."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    ok = j <= i
    if window:
        ok = ok & (i - j < window)
    return ok


def attention_weights(q: Tensor, k: Tensor, scale: float, cap: Optional[float], window: Optional[int]) -> Tensor:
    """q [T, H, dk], k [T, G, dk] (already unit-normed) -> softmax weights [H, T, T]."""
    T, H, _ = q.shape
    G = k.shape[1]
    k_of_head = k[:, torch.arange(H) // (H // G), :]  # head h reads key/value head floor(h / (H / G))
    s = torch.einsum("ihd,jhd->hij", q, k_of_head) * scale
    s = soft_cap(s, cap)
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(q.dtype)
    s = s - head_slopes(H, q.dtype)[:, None, None] * dist
    s = s.masked_fill(~visible(T, window)[None], float("-inf"))
    return torch.softmax(s, dim=-1)


def mix_heads(w: Tensor, talk: Tensor) -> Tensor:
    """w [H, T, T] -> w'[h] = sum_g talk[h, g] w[g]."""
    return torch.einsum("hg,gij->hij", talk, w)


def blend_values(v: Tensor, v_first: Optional[Tensor], lam: Optional[Tensor]) -> Tensor:
    return v if v_first is None else (1.0 - lam) * v + lam * v_first


def apply_weights(w: Tensor, v: Tensor) -> Tensor:
    """w [H, T, T], v [T, G, dv] -> [T, H, dv]; head h uses the values of its own key/value head."""
    H, G = w.shape[0], v.shape[1]
    return torch.einsum("hij,jhd->ihd", w, v[:, torch.arange(H) // (H // G), :])


def attention_mixer(h: Tensor, W: Dict[str, Tensor], p: str, m: dict, eps: float, v_first: Optional[Tensor]):
    """The whole mixer for input h [T, D]; returns (output [T, D], the values it used [T, G, dv])."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, dk)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, dk)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, dv)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    v = blend_values(v, v_first, W.get(p + "vmix"))
    window = (m.get("mask") or {}).get("size")
    w = attention_weights(q, k, m["scale"], m.get("softcap"), window)
    w = mix_heads(w, W[p + "talk"])
    o = apply_weights(w, v)
    o = o * torch.sigmoid(h @ W[p + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ W[p + "o"].T, v


def poly_norm(z: Tensor, c: Tensor, eps: float) -> Tensor:
    return c[0] * unit_rms(z, eps) + c[1] * unit_rms(z * z, eps) + c[2] * unit_rms(z * z * z, eps) + c[3]


def feed_forward(h: Tensor, W: Dict[str, Tensor], p: str, eps: float) -> Tensor:
    return poly_norm(h @ W[p + "up"].T, W[p + "act"], eps) @ W[p + "down"].T


def depth_average(results: List[Tensor], w: Tensor) -> Tensor:
    assert len(results) == w.numel()
    return sum(w[j] * results[j] for j in range(len(results)))


def plain_streams(W: Dict[str, Tensor], config: dict, tokens: Tensor) -> List[Tensor]:
    """The residual stream after every layer (what the next layer reads), [T, D] each."""
    eps = config["norm"]["eps"]
    x = W["embed"][tokens]
    results, out = [x], []
    v_first = None
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = rms_norm(x, W[p + "norm1"], eps)
        blending = bool(layer["mixer"].get("v_mix"))
        y, v = attention_mixer(h, W, p + "mix.", layer["mixer"], eps, v_first if blending else None)
        if blending and v_first is None:
            v_first = v
        if layer.get("mlp") is not None:
            y = y + feed_forward(h, W, p + "mlp.", eps)
        results.append(x + y)
        x = depth_average(results, W[p + "dwa"])
        out.append(x)
    return out


def plain_logits(W: Dict[str, Tensor], config: dict, tokens: Tensor) -> Tensor:
    x = plain_streams(W, config, tokens)[-1]
    return rms_norm(x, W["final.norm"], config["norm"]["eps"]) @ W["embed"].T


def plain_greedy(W: Dict[str, Tensor], config: dict, prompt: List[int], n_new: int) -> List[int]:
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(plain_logits(W, config, torch.tensor(toks))[-1])))
    return toks[len(prompt):]


def make_config(vocab=97, width=64, layers=None, eps=1e-5) -> dict:
    return {"architecture": "Zederax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def layer(heads=4, kv_heads=2, dim=16, vdim=8, window=24, scale=None, softcap=10.0, v_mix=True, ff=48) -> dict:
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 3.0 / math.sqrt(dim),
             "v_mix": v_mix}
    if softcap is not None:
        mixer["softcap"] = softcap
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def random_weights(config: dict, seed: int, dtype=torch.float64) -> Dict[str, Tensor]:
    """Weights drawn so that every mechanism matters: scores of order one before the cap, a mixing matrix far from the
    identity, blends between 0.2 and 0.8, depth weights of both signs. Values are bfloat16 numbers (a file stores them exactly)."""
    g = torch.Generator().manual_seed(seed)
    D, V = config["width"], config["vocab"]

    def n(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16).to(dtype)

    W = {"embed": n(V, D), "final.norm": 1 + n(D, std=0.2)}
    for i, L in enumerate(config["layers"]):
        m, p = L["mixer"], f"l{i}."
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        W[p + "norm1"] = 1 + n(D, std=0.2)
        for name, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
            W[p + "mix." + name] = n(rows, D, std=1 / math.sqrt(D))
            W[p + "mix." + name + ".b"] = n(rows, std=0.3)
        W[p + "mix.g"] = n(H, D, std=1 / math.sqrt(D))
        W[p + "mix.talk"] = (torch.eye(H) + torch.randn(H, H, generator=g) * 0.4).to(torch.bfloat16).to(dtype)
        W[p + "mix.o"] = n(D, H * dv, std=1 / math.sqrt(H * dv))
        if m.get("v_mix"):
            W[p + "mix.vmix"] = (0.2 + 0.6 * torch.rand((), generator=g)).to(torch.bfloat16).to(dtype)
        if L.get("mlp") is not None:
            F = L["mlp"]["ff"]
            W[p + "mlp.up"] = n(F, D, std=1 / math.sqrt(D))
            W[p + "mlp.down"] = n(D, F, std=1 / math.sqrt(F))
            W[p + "mlp.act"] = n(4, std=0.7)
        dwa = torch.randn(i + 2, generator=g) * 0.3
        dwa[-1] += 1.0
        W[p + "dwa"] = dwa.to(torch.bfloat16).to(dtype)
    return W


def write_folder(config: dict, W: Dict[str, Tensor], path: str, dtype=torch.bfloat16) -> str:
    """config.json and model.safetensors of these weights, through the safetensors package."""
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.to(dtype).contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return path
