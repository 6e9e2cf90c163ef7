"""Seeded synthetic q/k/v for the five benchmark workloads.

The workloads are not taken from the reference (its benchmark needs model
weights); they are defined here:

* ``text`` tokens: q, k, v ~ N(0,1) per element.  A rank-8 term is then added to
  both q and k: with C ~ N(0,1)^{H_kv x 8} and B ~ N(0,1)^{8 x d}, the matrix of
  per-head directions U = C B / sqrt(8) has rank 8; every token of KV head g -
  its keys and the queries of the query heads that read it - gets ``2.0 * U[g]``
  added.  Finally rotary position embedding, rotate-half form, base 500000,
  positions 0..L-1, on q and k.  Before the rotation all queries and keys of a
  head share the direction, so q.k carries a positive common term; the rotation
  makes that term a function of the distance between the tokens, largest at
  distance 0 and falling off roughly like a power of the distance whose
  exponent grows with |U[g]|^2 - heads differ from sharply local to
  heavy-tailed.  (The first key block is always kept by the selection rule.)
* ``video`` tokens (workload 3): per frame of 256 tokens a mean vector ~ N(0,1)
  plus N(0, 0.3^2) per-token noise, drawn independently for q, k and v; the
  same rotary embedding on q and k.
* ``field`` tokens (workload 4): a T x H x W = 33 x 45 x 80 grid; white noise
  filtered by a first-order autoregression with rho = exp(-1/2) along each
  axis (separable exponential correlation, length 2, unit variance), plus
  N(0,1) noise, drawn independently for q, k, v; no rotary embedding.

Everything is generated in fp32 on the requested device from one
``torch.Generator`` seed, head by head, then cast to the requested dtype, so a
CPU oracle and the GPU path can be fed bit-identical tensors.
"""
import math
from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    L: int
    heads: int
    kv_heads: int
    stride: int
    threshold: float
    chunk_size: object  # int or None (operator default)
    causal: bool
    kind: str           # "text" | "video+text" | "field+text"
    dtype: torch.dtype = torch.bfloat16


WORKLOADS = [
    Workload("cfg0_cpu_L4096_mha32_S8", 4096, 32, 32, 8, 0.9, 2048, True, "text", torch.float32),
    Workload("cfg1_llama8b_L32768_gqa32x8_S8", 32768, 32, 8, 8, 0.9, 16384, True, "text"),
    Workload("cfg2_llama8b_L131072_gqa32x8_S16", 131072, 32, 8, 16, 0.9, 16384, True, "text"),
    Workload("cfg3_qwen2vl_L65536_gqa28x4_S16", 65536, 28, 4, 16, 0.9, None, True, "video+text"),
    Workload("cfg4_hunyuan_L119056_mha24_S8", 119056, 24, 24, 8, 0.95, None, False, "field+text"),
]

ROPE_BASE = 500000.0
D = 128


def _rope_tables(L, device):
    inv = ROPE_BASE ** (-torch.arange(0, D, 2, dtype=torch.float32, device=device) / D)
    ang = torch.arange(L, dtype=torch.float32, device=device)[:, None] * inv[None, :]
    ang = torch.cat([ang, ang], dim=-1)
    return ang.cos(), ang.sin()


def _rope(x, cos, sin):
    x1, x2 = x[..., : D // 2], x[..., D // 2 :]
    return x * cos + torch.cat([-x2, x1], dim=-1) * sin


def _randn(shape, gen, device):
    return torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


def _ar1(x, dim, rho):
    """Unit-variance first-order autoregression along ``dim`` (in place)."""
    n = x.shape[dim]
    gain = math.sqrt(1.0 - rho * rho)
    prev = x.select(dim, 0)
    for i in range(1, n):
        cur = x.select(dim, i)
        cur.mul_(gain).add_(prev, alpha=rho)
        prev = cur
    return x


def make_inputs(w: Workload, device="cpu", seed=0, L=None, heads=None, kv_heads=None, dtype=None, rank8="head"):
    """q [1,H,L,128], k, v [1,H_kv,L,128] for a workload (optionally shrunk).

    ``rank8`` chooses the reading of the text workloads' "shared rank-8 Gaussian
    component": "head" (default) is the per-KV-head direction described above;
    "token" draws a coefficient vector c_t ~ N(0, I_8) per TOKEN instead and adds
    ``2.0 * c_t B / sqrt(8)`` to that token's query (every head) and key (every
    KV head) - shared between q and k of a token, not along the sequence, which
    gives diffuse attention without locality (kept as the dense end of the
    benchmark's density sweep)."""
    L = w.L if L is None else L
    H = w.heads if heads is None else heads
    Hkv = w.kv_heads if kv_heads is None else kv_heads
    dtype = w.dtype if dtype is None else dtype
    group = H // Hkv
    gen = torch.Generator(device=device).manual_seed(seed)
    q = torch.empty((1, H, L, D), dtype=dtype, device=device)
    k = torch.empty((1, Hkv, L, D), dtype=dtype, device=device)
    v = torch.empty((1, Hkv, L, D), dtype=dtype, device=device)

    if w.kind == "field+text":
        T, Hh, Ww = 33, 45, 80
        n_field = T * Hh * Ww
        if L != w.L:  # shrink the time axis for reduced-size runs
            T = max(1, int(round(T * L / w.L)))
            n_field = min(L, T * Hh * Ww)
        rho = math.exp(-0.5)

        def field_tokens():
            f = _randn((T, Hh, Ww, D), gen, device)
            for dim in range(3):
                _ar1(f, dim, rho)
            f = f.reshape(-1, D)[:n_field]
            out = _randn((L, D), gen, device)
            out[:n_field] += f
            return out

        for h in range(H):
            q[0, h] = field_tokens().to(dtype)
        for h in range(Hkv):
            k[0, h] = field_tokens().to(dtype)
            v[0, h] = field_tokens().to(dtype)
        return q, k, v

    cos, sin = _rope_tables(L, device)
    n_video = 0
    if w.kind == "video+text":
        frames = 240 if L == w.L else max(1, (L * 240 // w.L))
        n_video = min(L, frames * 256)
    if rank8 not in ("head", "token"):
        raise ValueError("rank8 must be 'head' or 'token'")
    coeff = _randn((Hkv, 8), gen, device)
    basis = _randn((8, D), gen, device)
    direction = 2.0 * (coeff @ basis) / math.sqrt(8.0)   # [Hkv, D], rank 8, shared by q and k
    per_token = 2.0 * (_randn((L, 8), gen, device) @ basis) / math.sqrt(8.0) if rank8 == "token" else None

    def tokens(kv_head, shared):
        x = _randn((L, D), gen, device)
        if shared:
            x[n_video:] += direction[kv_head] if per_token is None else per_token[n_video:]
        if n_video:
            nf = (n_video + 255) // 256
            means = _randn((nf, D), gen, device).repeat_interleave(256, dim=0)[:n_video]
            x[:n_video] = means + 0.3 * x[:n_video]
        return x

    for h in range(H):
        q[0, h] = _rope(tokens(h // group, True), cos, sin).to(dtype)
    for g in range(Hkv):
        k[0, g] = _rope(tokens(g, True), cos, sin).to(dtype)
        v[0, g] = tokens(g, False).to(dtype)
    return q, k, v
