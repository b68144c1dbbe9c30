"""Latent attention and the pieces of parallel layers on a float32 residual stream.

Latent attention caches ONE small vector per token and layer: the RMS-normed latent ``c`` [rank] of
which every head's keys and values are up-projections (k_h = Wuk_h c, v_h = Wuv_h c), and optionally
a single rotary key slice [rot_dim] that every head uses.  Head h's score of query i against key j is
(q_h,i . Wuk_h c_j + qrot_h,i . krot_j) * scale.  The key up-projection is folded into the query,
q~_h = Wuk_h^T q_h, and the value up-projection is applied after the weighted sum, so attention runs
over a single shared K/V head whose keys are [c | krot] and whose values are c:
:func:`~.seqmix.window_attention` with G = 1 (its ``sinks`` argument gives the softmax a learned
per-head denominator term).  The paged cache holds the latent in the two layouts that kernel reads:
k [NB, 1, BS, rank + rot_dim] and v [NB, 1, rank, BS].

Same dispatch as the other ops: CUDA tensors go to the in-tree HIP kernels (csrc/kernels/latent.hip)
and raise if those are not built; CPU tensors run the plain PyTorch forms.  Activations are bfloat16
or float32; norms, angles, gates, scores and softmax weights are float32 in both.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import seqmix as sm
from .seqmix import SeqBatch, _ck, _f32flag, _k, _ptr, _stream


FOLD_MAX_TOKENS = 64      # up to this many tokens the per-head products run in the fold / unfold kernels


@dataclass
class LatentSpec:
    """Sizes and constants of one latent-attention mixer."""
    heads: int
    dim: int                 # unrotated query / key dimensions per head
    vdim: int                # value dimensions per head
    rank: int                # key / value latent size
    q_rank: int              # query latent size
    scale: float
    rot_dim: int = 0         # rotated query / key dimensions per head (one key slice serves every head)
    gated: bool = False      # per-head sigmoid output gate (one more row per head in the down projection)

    @property
    def key_width(self) -> int:
        return self.rank + self.rot_dim

    @property
    def down_width(self) -> int:
        return self.q_rank + self.rank + self.rot_dim + (self.heads if self.gated else 0)


def latent_prep(down: torch.Tensor, spec: LatentSpec, q_norm: torch.Tensor, c_norm: torch.Tensor,
                freqs: Optional[torch.Tensor], eps: float, k_cache: torch.Tensor, v_cache: torch.Tensor,
                slot_mapping: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """From the fused down projection ``down`` [T, q_rank | rank | rot_dim | ...]: the RMS-normed query
    latent (returned, [T, q_rank]); the RMS-normed key/value latent and the shared key part, rotated in
    interleaved pairs (2i, 2i + 1) by ``position * freqs[i]``, appended at ``slot_mapping`` to
    k_cache [NB, 1, BS, rank + rot_dim] and v_cache [NB, 1, rank, BS]."""
    t = down.shape[0]
    qr, r, dr = spec.q_rank, spec.rank, spec.rot_dim
    if down.shape[1] < qr + r + dr or k_cache.shape[3] != r + dr or v_cache.shape[2] != r:
        raise ValueError("latent_prep: shape mismatch")
    nf = 0 if freqs is None else freqs.numel()
    bs = k_cache.shape[2]
    if not down.is_cuda:
        x = down.float()
        cq = sm._ref_rms(x[:, :qr], q_norm, eps, 0.0).to(down.dtype)
        c = sm._ref_rms(x[:, qr:qr + r], c_norm, eps, 0.0)
        rows = [c]
        if dr:
            kr = x[:, qr + r:qr + r + dr]
            rows.append(sm._ref_rope_interleaved(kr[:, None, :], positions, freqs, 1.0)[:, 0] if nf else kr)
        key = torch.cat(rows, -1).to(k_cache.dtype)
        slot = slot_mapping.long()
        k_cache[slot // bs, 0, slot % bs] = key
        v_cache[slot // bs, 0, :, slot % bs] = key[:, :r]
        return cq
    _ck(down, "down")
    _ck(k_cache, "k_cache", down.dtype)
    _ck(v_cache, "v_cache", down.dtype)
    _ck(q_norm, "q_norm", down.dtype)
    _ck(c_norm, "c_norm", down.dtype)
    if q_norm.numel() != qr or c_norm.numel() != r or k_cache.shape[1] != 1 or v_cache.shape[3] != bs:
        raise ValueError("latent_prep: weight / cache shape")
    if freqs is not None:
        _ck(freqs, "freqs", torch.float32)
    cq = torch.empty(t, qr, dtype=down.dtype, device=down.device)
    _k().lat_prep(cq.data_ptr(), down.data_ptr(), down.shape[1], 0, qr, q_norm.data_ptr(), qr, r, c_norm.data_ptr(),
                  qr + r, dr, _ptr(freqs), nf, positions.data_ptr(), slot_mapping.data_ptr(), k_cache.data_ptr(),
                  v_cache.data_ptr(), bs, float(eps), t, _f32flag(down), _stream())
    return cq


def latent_queries(q: torch.Tensor, w_uk: torch.Tensor, spec: LatentSpec, freqs: Optional[torch.Tensor],
                   positions: torch.Tensor) -> torch.Tensor:
    """q [T, H * (dim + rot_dim)] -> q~ [T, H, rank + rot_dim]: per head the unrotated part times
    ``w_uk`` [H, dim, rank] (the key up-projection folded into the query) next to the rotated part."""
    t = q.shape[0]
    h, d, dr, r = spec.heads, spec.dim, spec.rot_dim, spec.rank
    nf = 0 if freqs is None else freqs.numel()
    if q.is_cuda and t <= FOLD_MAX_TOKENS:
        # few tokens: product, rotation and concatenation in one launch
        _ck(q, "q")
        _ck(w_uk, "w_uk", q.dtype)
        out = torch.empty(t, h, r + dr, dtype=q.dtype, device=q.device)
        _k().lat_q_fold(out.data_ptr(), q.data_ptr(), w_uk.data_ptr(), t, h, r, d, dr, _ptr(freqs), nf,
                        positions.data_ptr(), _f32flag(q), _stream())
        return out
    q3 = q.view(t, h, d + dr)
    qa = torch.bmm(q3[:, :, :d].transpose(0, 1), w_uk)                    # [H, T, rank]
    if not q.is_cuda:
        parts = [qa.transpose(0, 1)]
        if dr:
            qr = q3[:, :, d:].float()
            parts.append((sm._ref_rope_interleaved(qr, positions, freqs, 1.0) if nf else qr).to(q.dtype))
        return torch.cat(parts, -1).contiguous()
    _ck(q, "q")
    out = torch.empty(t, h, r + dr, dtype=q.dtype, device=q.device)
    _k().lat_q_pack(out.data_ptr(), qa.data_ptr(), q.data_ptr(), t, h, r, d, dr, _ptr(freqs), nf, positions.data_ptr(),
                    _f32flag(q), _stream())
    return out


def latent_values(o_lat: torch.Tensor, w_uv_t: torch.Tensor, gate: Optional[torch.Tensor] = None,
                  gate_col: int = 0) -> torch.Tensor:
    """o_lat [T, H, rank] (softmax-weighted sums of latents) -> [T, H * vdim]: per head times
    ``w_uv_t`` [H, rank, vdim], then times sigmoid(gate[t, gate_col + h]) when ``gate`` (a [T, *] tensor
    holding one gate logit per head from column ``gate_col``) is given."""
    t, h, r = o_lat.shape
    vd = w_uv_t.shape[2]
    if o_lat.is_cuda and t <= FOLD_MAX_TOKENS:
        # few tokens: product, gate and the [T, H vdim] layout in one launch
        _ck(o_lat, "o_lat")
        _ck(w_uv_t, "w_uv_t", o_lat.dtype)
        if gate is not None:
            _ck(gate, "gate", o_lat.dtype)
        out = torch.empty(t, h * vd, dtype=o_lat.dtype, device=o_lat.device)
        gp = 0 if gate is None else gate.data_ptr() + gate_col * gate.element_size()
        _k().lat_v_unfold(out.data_ptr(), o_lat.data_ptr(), w_uv_t.data_ptr(), gp, 0 if gate is None else gate.shape[1],
                          t, h, r, vd, _f32flag(o_lat), _stream())
        return out
    o = torch.bmm(o_lat.transpose(0, 1), w_uv_t)                          # [H, T, vdim]
    if not o_lat.is_cuda:
        o = o.transpose(0, 1).float()
        if gate is not None:
            o = o * torch.sigmoid(gate[:, gate_col:gate_col + h].float())[:, :, None]
        return o.reshape(t, h * vd).to(o_lat.dtype)
    out = torch.empty(t, h * vd, dtype=o_lat.dtype, device=o_lat.device)
    if gate is not None:
        _ck(gate, "gate", o_lat.dtype)
    gp = 0 if gate is None else gate.data_ptr() + gate_col * gate.element_size()
    _k().lat_head_gate(out.data_ptr(), o.data_ptr(), gp, 0 if gate is None else gate.shape[1], t, h, vd,
                       _f32flag(o_lat), _stream())
    return out


def latent_attention(h: torch.Tensor, w: dict, spec: LatentSpec, freqs: Optional[torch.Tensor], eps: float,
                     k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                     block_tables: torch.Tensor, sb: SeqBatch, num_decode: Optional[int] = None,
                     window: int = 1 << 30, max_ctx: Optional[int] = None) -> torch.Tensor:
    """The whole mixer on a varlen batch.  ``w``: ``down`` [q_rank + rank + rot_dim (+ H), W] (query
    latent | key/value latent | shared key part | gates), ``q_norm``, ``c_norm``, ``uq``
    [H (dim + rot_dim), q_rank], ``uk`` [H, dim, rank], ``uv_t`` [H, rank, vdim], ``o`` [W, H vdim] and
    optionally ``sinks`` [H] float32.  Returns [T, W]."""
    from . import linear
    down = linear(h, w["down"])
    cq = latent_prep(down, spec, w["q_norm"], w["c_norm"], freqs, eps, k_cache, v_cache, slot_mapping, sb.positions)
    qf = latent_queries(linear(cq, w["uq"]), w["uk"], spec, freqs, sb.positions)
    o_lat = sm.window_attention(qf, k_cache, v_cache, block_tables, sb, window, spec.scale, num_decode=num_decode,
                                sinks=w.get("sinks"), max_ctx=max_ctx)
    o = latent_values(o_lat, w["uv_t"], down if spec.gated else None, spec.q_rank + spec.rank + spec.rot_dim)
    return linear(o, w["o"])


# ------------------------------------------------------------------ parallel layers on a float32 stream
def par_add(x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None, rounded: bool = False):
    """x += a + b in place on the float32 stream (both sublayers of a parallel layer at once).  With
    ``rounded`` also returns the new stream in ``a``'s dtype (the input of a following projection)."""
    if not x.is_cuda:
        x.add_(a.float() if b is None else a.float() + b.float())
        return x, (x.to(a.dtype) if rounded else None)
    _ck(x, "x", torch.float32)
    _ck(a, "a")
    if a.shape != x.shape or (b is not None and (b.shape != x.shape or b.dtype != a.dtype or not b.is_contiguous())):
        raise ValueError("par_add: shape / dtype mismatch")
    xr = None
    if rounded:
        xr = x if a.dtype == torch.float32 else torch.empty_like(a)
    _k().par_add(x.data_ptr(), a.data_ptr(), _ptr(b), 0 if xr is None or xr is x else xr.data_ptr(), x.numel(),
                 _f32flag(a), _stream())
    return x, xr


def stream_cat(x: torch.Tensor, x0: torch.Tensor, act_dtype) -> torch.Tensor:
    """[x | x0] [T, 2 W] in ``act_dtype`` from two float32 streams."""
    if not x.is_cuda:
        return torch.cat([x, x0], -1).to(act_dtype)
    _ck(x, "x", torch.float32)
    _ck(x0, "x0", torch.float32)
    if x.shape != x0.shape:
        raise ValueError("stream_cat: shape mismatch")
    out = torch.empty(x.shape[0], 2 * x.shape[1], dtype=act_dtype, device=x.device)
    _k().stream_cat(out.data_ptr(), x.data_ptr(), x0.data_ptr(), x.shape[0], x.shape[1], _f32flag(out), _stream())
    return out


def stream_set(a: torch.Tensor) -> torch.Tensor:
    """A new float32 stream holding ``a``."""
    if not a.is_cuda or a.dtype == torch.float32:
        return a.float()
    _ck(a, "a")
    x = torch.empty(a.shape, dtype=torch.float32, device=a.device)
    _k().stream_set(x.data_ptr(), a.data_ptr(), a.numel(), _f32flag(a), _stream())
    return x


def linear_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T), W = [Wg; Wu]: in the GEMM epilogue where the framework's bf16 GEMMs take
    the shape, else the projection followed by the gate kernel (float32, odd sizes)."""
    from . import linear, linear_swiglu as fused
    n = w_gate_up.shape[0]
    if not x.is_cuda or (x.dtype == torch.bfloat16 and n % 256 == 0 and x.shape[-1] % 64 == 0):
        return fused(x, w_gate_up)
    gu = linear(x, w_gate_up)
    _ck(gu, "gu")
    out = torch.empty(gu.shape[0], n // 2, dtype=gu.dtype, device=gu.device)
    _k().silu_glu(out.data_ptr(), gu.data_ptr(), gu.shape[0], n // 2, _f32flag(gu), _stream())
    return out


def side_gate(z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, col: int) -> torch.Tensor:
    """gelu_tanh(z) * table[ids, col : col + dim] for z [T, dim]: a per-token vector looked up in a side
    table, gated by a projection of the stream."""
    t, dim = z.shape
    if not z.is_cuda:
        e = table.index_select(0, ids.long())[:, col:col + dim].float()
        return (sm.gelu_tanh_f32(z.float()) * e).to(z.dtype)
    _ck(z, "z")
    _ck(table, "table", z.dtype)
    _ck(ids, "ids", torch.int32)
    if col < 0 or col + dim > table.shape[1]:
        raise ValueError("side_gate: columns outside the table")
    g = torch.empty_like(z)
    _k().side_gate(g.data_ptr(), z.data_ptr(), table.data_ptr(), ids.data_ptr(), t, table.shape[0], table.shape[1], col,
                   dim, _f32flag(z), _stream())
    return g
