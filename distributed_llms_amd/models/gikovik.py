"""Gikovik: a layer-list decoder of PARALLEL layers with latent attention, dense or mixture-of-experts
feed-forwards, a per-layer token input and a looped span of layers.

``config.json`` keys (read by ``config._from_gikovik``): ``width``, ``vocab``, ``norm.eps``,
``token_side.dim``, ``loop`` (``start``, ``stop``, ``times``) and ``layers``: per layer ``type``
("latent_attention" | "latent_attention_2"), ``mixer`` and ``mlp``.

  mixer: ``heads``, ``dim`` (unrotated q / k size per head), ``vdim``, ``kv_rank`` (latent size), ``q_rank``
      (query latent size), ``scale``; "latent_attention" adds a learned per-head sink to the softmax
      denominator; "latent_attention_2" has ``rot_dim`` more query dimensions per head that meet a
      single rotary key slice common to every head (``rot``: ``base``, ``dims``; interleaved pairs) and a per-head
      sigmoid output gate.
  mlp: None, {"kind": "dense", "ff"} (SwiGLU) or {"kind": "moe", "expert": {"ff"}, "router": {"experts",
      "top", "scale", "groups": {"count", "keep"}}, "shared": {"ff"} | None} (squared-ReLU experts
      down(relu(up h)^2), sigmoid scores, a choice bias, groups of neighbouring experts, a gated
      shared expert).

One layer: h = rms(x) w1;  x += mixer(h) + ff(h);  then the token input
x += rms(P (gelu_tanh(G x) * e_tok)) w_s with e_tok the layer's ``token_side.dim`` columns of a second
embedding table.  Layers [loop.start, loop.stop) are repeated ``loop.times`` times back to back, sharing their
weights; every repetition starts with x <- W_in [x | x0] (x0: the token embedding) and gets separate caches.

Checkpoint names: ``embed``, ``side.embed``, ``loop.in``, ``final.norm``, ``head``; per layer ``l<i>.``:
``norm1``; ``mix.dq`` (+ ``.norm``), ``mix.uq``, ``mix.dkv`` (+ ``.norm``), ``mix.uk``, ``mix.uv``, ``mix.o``,
``mix.sink`` or ``mix.g``; ``mlp.gate|up|down`` or ``mlp.router``, ``mlp.correction``, ``mlp.e<j>.up|down``,
``mlp.shared.up|down|sg``; ``side.gate|proj|norm``.  Linear weights are [out, in].

What a sequence keeps between steps is paged only: per layer RUN (a looped layer counts once per
pass) the key/value latent and the shared rotated key part of every token, in the two layouts the
attention kernels read (ops/latent.py).  The residual stream, norms, rotation angles, router, scores
and softmax weights are float32 also when activations are bfloat16.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch

from .. import ops
from ..config import ModelConfig
from ..ops import latent as lat
from ..ops import moe
from ..ops import seqmix as sm
from .hybrid import LayerListStage
from .stage import BatchMeta
from .weights import tensor_seed

MIXERS = ("latent_attention", "latent_attention_2")


def latent_spec(layer: Dict[str, Any]) -> lat.LatentSpec:
    m = layer["mixer"]
    rot = layer["type"] == "latent_attention_2"
    return lat.LatentSpec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), rank=int(m["kv_rank"]),
                          q_rank=int(m["q_rank"]), scale=float(m["scale"]), rot_dim=int(m["rot_dim"]) if rot else 0,
                          gated=rot)


def layer_runs(cfg: ModelConfig) -> List[Tuple[int, bool]]:
    """[(layer index, the run enters a pass of the loop)] in execution order."""
    n = len(cfg.layers)
    lp = cfg.loop
    if not lp:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(lp["start"])]
    for _ in range(lp["times"]):
        runs += [(i, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, False) for i in range(lp["stop"], n)]


def layer_shapes(width: int, layer: Dict[str, Any], side_dim: int) -> Dict[str, tuple]:
    """Checkpoint tensor name (without the ``l<i>.`` prefix) -> shape."""
    sp = latent_spec(layer)
    s: Dict[str, tuple] = {
        "norm1": (width,), "mix.dq": (sp.q_rank, width), "mix.dq.norm": (sp.q_rank,),
        "mix.uq": (sp.heads * (sp.dim + sp.rot_dim), sp.q_rank), "mix.dkv": (sp.rank + sp.rot_dim, width),
        "mix.dkv.norm": (sp.rank,), "mix.uk": (sp.heads * sp.dim, sp.rank), "mix.uv": (sp.heads * sp.vdim, sp.rank),
        "mix.o": (width, sp.heads * sp.vdim)}
    if sp.gated:
        s["mix.g"] = (sp.heads, width)
    else:
        s["mix.sink"] = (sp.heads,)
    mlp = layer.get("mlp")
    if mlp and mlp["kind"] == "dense":
        s.update({"mlp.gate": (mlp["ff"], width), "mlp.up": (mlp["ff"], width), "mlp.down": (width, mlp["ff"])})
    elif mlp:
        e, f = mlp["router"]["experts"], mlp["expert"]["ff"]
        s.update({"mlp.router": (e, width), "mlp.correction": (e,)})
        for j in range(e):
            s.update({f"mlp.e{j}.up": (f, width), f"mlp.e{j}.down": (width, f)})
        if mlp.get("shared"):
            fs = mlp["shared"]["ff"]
            s.update({"mlp.shared.up": (fs, width), "mlp.shared.down": (width, fs), "mlp.shared.sg": (1, width)})
    if side_dim:
        s.update({"side.gate": (side_dim, width), "side.proj": (width, side_dim), "side.norm": (width,)})
    return s


def model_shapes(cfg: ModelConfig) -> Dict[str, tuple]:
    w, sd = cfg.hidden_size, cfg.token_side_dim
    s = {"embed": (cfg.vocab_size, w), "final.norm": (w,), "head": (cfg.vocab_size, w)}
    if sd:
        s["side.embed"] = (cfg.vocab_size, sd * len(cfg.layers))
    if cfg.loop:
        s["loop.in"] = (w, 2 * w)
    for i, layer in enumerate(cfg.layers):
        s.update({f"l{i}.{n}": shp for n, shp in layer_shapes(w, layer, sd).items()})
    return s


def synth_state_dict(cfg: ModelConfig, seed: int = 0, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Seeded random weights under the checkpoint names (CPU): projections ~ N(0, 1 / fan_in), norm
    weights around one, sinks, corrections and the router spread so that choices are not close calls."""
    sd = {}
    for name, shape in model_shapes(cfg).items():
        g = torch.Generator().manual_seed(tensor_seed(seed, 0, name))
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm", "norm1") or name == "final.norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "sink":
            t = torch.randn(shape, generator=g)
        elif leaf == "correction":
            t = 0.3 * torch.randn(shape, generator=g)
        elif leaf == "router":
            t = 3.0 * torch.randn(shape, generator=g) / shape[-1] ** 0.5
        elif name in ("embed", "side.embed"):
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
        sd[name] = t.to(dtype)
    return sd


class GikovikStage(LayerListStage):
    """All layers of a Gikovik model on one device (see the module docstring)."""

    @staticmethod
    def layer_param_count(width: int, layer: Dict[str, Any]) -> int:
        return sum(int(torch.Size(s).numel()) for s in layer_shapes(width, layer, 0).values())

    @staticmethod
    def kv_elements_per_token(cfg: ModelConfig) -> int:
        # the latent is held twice (row-major for the scores, transposed for the weighted sum)
        return sum(2 * sp.rank + sp.rot_dim for sp in (latent_spec(cfg.layers[i]) for i, _ in layer_runs(cfg)))

    def __init__(self, cfg: ModelConfig, layer_start: int = 0, layer_end: Optional[int] = None, device="cpu",
                 dtype=torch.bfloat16, units: Optional[tuple] = None, tp=None, unit_group: int = 2):
        super().__init__(cfg, layer_start, layer_end, device, dtype, units, tp, unit_group)
        self.runs = layer_runs(cfg)
        self.lspec = [latent_spec(l) for l in self.specs]
        self.freqs: Dict[int, Optional[torch.Tensor]] = {}
        for i, (l, sp) in enumerate(zip(self.specs, self.lspec)):
            if l["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unsupported type {l['type']!r}")
            self.freqs[i] = None
            if sp.rot_dim:
                r = l["mixer"]["rot"]
                if r["dims"] % 2 or r["dims"] > sp.rot_dim:
                    raise ValueError(f"layer {i}: rot.dims does not fit rot_dim")
                self.freqs[i] = sm.yarn_frequencies(int(r["dims"]), float(r["base"]), None)[0].to(self.device)
            mlp = l.get("mlp")
            if mlp and mlp["kind"] == "moe":
                r = mlp["router"]
                g = r.get("groups") or {"count": 1, "keep": 1}
                if r["experts"] % g["count"] or g["keep"] > g["count"] or g["keep"] * (r["experts"] // g["count"]) < r["top"]:
                    raise ValueError(f"layer {i}: expert groups do not fit")

    # ------------------------------------------------------------------ weights
    def load_hf_state(self, sd: Dict[str, torch.Tensor]) -> "GikovikStage":
        """From checkpoint-named tensors: fuses dq | dkv | g into one down projection and gate | up, stacks
        the experts, stores uk as [H, dim, rank] and uv transposed ([H, rank, vdim]); what feeds float32
        math directly (router rows with the shared expert's gate row, corrections, sinks) is float32."""
        want = model_shapes(self.cfg)
        for n, shp in want.items():
            if n not in sd:
                raise KeyError(f"checkpoint lacks {n}")
            if tuple(sd[n].shape) != tuple(shp):
                raise ValueError(f"{n}: shape {tuple(sd[n].shape)}, config says {tuple(shp)}")
        cv = lambda t: t.to(device=self.device, dtype=self.dtype).contiguous()
        f32 = lambda t: t.to(device=self.device, dtype=torch.float32).contiguous()
        self.embed = {"embed": cv(sd["embed"])}
        if self.cfg.token_side_dim:
            self.embed["side"] = cv(sd["side.embed"])
        if self.cfg.loop:
            self.embed["loop_in"] = cv(sd["loop.in"])
        self.head = {"final_norm": cv(sd["final.norm"]), "lm_head": cv(sd["head"])}
        self.layers = []
        for i, (layer, sp) in enumerate(zip(self.specs, self.lspec)):
            p = f"l{i}."
            parts = [sd[p + "mix.dq"], sd[p + "mix.dkv"]] + ([sd[p + "mix.g"]] if sp.gated else [])
            mix = {"down": cv(torch.cat(parts, 0)), "q_norm": cv(sd[p + "mix.dq.norm"]),
                   "c_norm": cv(sd[p + "mix.dkv.norm"]), "uq": cv(sd[p + "mix.uq"]),
                   "uk": cv(sd[p + "mix.uk"].view(sp.heads, sp.dim, sp.rank)),
                   "uv_t": cv(sd[p + "mix.uv"].view(sp.heads, sp.vdim, sp.rank).transpose(1, 2)),
                   "o": cv(sd[p + "mix.o"])}
            if not sp.gated:
                mix["sinks"] = f32(sd[p + "mix.sink"])
            w: Dict[str, Any] = {"norm1": cv(sd[p + "norm1"]), "mix": mix}
            mlp = layer.get("mlp")
            if mlp and mlp["kind"] == "dense":
                w["w_gu"] = cv(torch.cat([sd[p + "mlp.gate"], sd[p + "mlp.up"]], 0))
                w["w_down"] = cv(sd[p + "mlp.down"])
            elif mlp:
                e = mlp["router"]["experts"]
                rows = [sd[p + "mlp.router"]] + ([sd[p + "mlp.shared.sg"]] if mlp.get("shared") else [])
                w["router"] = f32(torch.cat(rows, 0))
                w["correction"] = f32(sd[p + "mlp.correction"])
                w["e_up"] = cv(torch.stack([sd[p + f"mlp.e{j}.up"] for j in range(e)], 0))
                w["e_down"] = cv(torch.stack([sd[p + f"mlp.e{j}.down"] for j in range(e)], 0))
                if mlp.get("shared"):
                    w["s_up"], w["s_down"] = cv(sd[p + "mlp.shared.up"]), cv(sd[p + "mlp.shared.down"])
            if self.cfg.token_side_dim:
                w["side_gate"], w["side_proj"] = cv(sd[p + "side.gate"]), cv(sd[p + "side.proj"])
                w["side_norm"] = cv(sd[p + "side.norm"])
            self.layers.append(w)
        return self

    def init_synthetic(self, seed: int = 0) -> "GikovikStage":
        return self.load_hf_state(synth_state_dict(self.cfg, seed))

    # ------------------------------------------------------------------ cache
    def cache_shapes(self, block_size: int) -> Dict[Any, tuple]:
        """One cache per layer run: k [NB, 1, BS, rank + rot_dim] (latent | shared rotated key part),
        v [NB, 1, rank, BS] (the latent again, transposed inside a block)."""
        out = {}
        for r, (i, _) in enumerate(self.runs):
            sp = self.lspec[i]
            out[r] = ((1, block_size, sp.key_width), (1, sp.rank, block_size))
        return out

    @property
    def graph_capturable(self) -> bool:
        """Whether a decode step runs without a host round trip.  Experts whose sizes the grouped
        kernels do not take (and float32) read the per-expert row counts on the host, which a HIP-graph
        capture cannot record: such a model decodes with eager launches."""
        for l in self.specs:
            mlp = l.get("mlp")
            if mlp and mlp["kind"] == "moe" and (self.dtype != torch.bfloat16 or self.cfg.hidden_size % 128
                                                 or mlp["expert"]["ff"] % 128):
                return False
        return True

    def allocate_state(self, num_slots: int):
        self.num_state_slots = num_slots
        self.state = []
        return self.state

    # ------------------------------------------------------------------ forward
    def _ff(self, h: torch.Tensor, w, mlp) -> torch.Tensor:
        if mlp["kind"] == "dense":
            return ops.linear(lat.linear_swiglu(h, w["w_gu"]), w["w_down"])
        r = mlp["router"]
        g = r.get("groups") or {"count": 1, "keep": 1}
        return moe.grouped_choice_ffn(h, w["router"], w["correction"], w["e_up"], w["e_down"], int(r["top"]),
                                      int(g["count"]), int(g["keep"]), float(r["scale"]), w.get("s_up"),
                                      w.get("s_down"))

    @torch.inference_mode()
    def forward(self, inp: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        if self.kv is None:
            raise RuntimeError("allocate_kv() before forward()")
        cfg = self.cfg
        eps, sdim = cfg.norm_eps, cfg.token_side_dim
        sb = self._seq_batch(meta)
        nd = meta.num_decode if meta.is_prefill else meta.num_seqs
        x0 = sm.embedding_f32(inp, self.embed["embed"])
        x = x0.clone() if cfg.loop else x0
        h = None                        # norm1 of the coming layer, when the previous layer's close made it
        last = len(self.runs) - 1
        for r, (i, enters) in enumerate(self.runs):
            spec, w = self.specs[i], self.layers[i]
            if enters:
                x = lat.stream_set(ops.linear(lat.stream_cat(x, x0, self.dtype), self.embed["loop_in"]))
                h = None
            if h is None:
                h = sm.rms_norm_f32(x, w["norm1"], eps, self.dtype, one_plus=False)
            kc, vc = self.kv.caches[r]
            a = lat.latent_attention(h, w["mix"], self.lspec[i], self.freqs[i], eps, kc, vc, meta.slot_mapping,
                                     meta.block_tables, sb, num_decode=nd,
                                     max_ctx=meta.max_ctx_d if (meta.is_prefill and nd) else meta.max_ctx)
            f = self._ff(h, w, spec["mlp"]) if spec.get("mlp") else None
            x, xr = lat.par_add(x, a, f, rounded=bool(sdim))
            h = None
            if sdim:
                z = lat.side_gate(ops.linear(xr, w["side_gate"]), self.embed["side"], inp, i * sdim)
                nxt = None
                if r < last and not self.runs[r + 1][1]:
                    nxt = self.layers[self.runs[r + 1][0]]["norm1"]
                x, h = sm.post_norm_add(x, ops.linear(z, w["side_proj"]), w["side_norm"], eps, 1.0, w_next=nxt,
                                        one_plus=False)
            if self.taps is not None:
                self.taps.append(x.clone())
        if meta.logits_idx is not None:
            x = x.index_select(0, meta.logits_idx)
        hf = sm.rms_norm_f32(x, self.head["final_norm"], eps, self.dtype, one_plus=False)
        return sm.softcap_f32(ops.linear(hf, self.head["lm_head"]), 0.0)
