"""Layer-list decoder ("Tudilix"): every layer names its own token mixer -- sliding-window attention
or a real-gated linear recurrent unit (RG-LRU) -- and an optional clipped-GLU feed-forward, around a
float32 residual stream with an RMS norm before AND after every sublayer.

``config.json`` keys (read by :func:`distributed_llms_amd.config.ModelConfig.from_layer_list`):
``width``, ``vocab``, ``norm.eps``, ``residual_mult``, ``logit_softcap`` and ``layers``: per layer
``type`` ("attention" | "rglru"), ``mixer`` and ``mlp`` (None, or ``kind`` "dense", ``ff``, ``limit``).

  attention mixer: ``heads``, ``kv_heads``, ``dim`` (q / k head size), ``vdim`` (v head size), ``conv``
      (taps of the causal convolution on every q / k / v channel), ``rot`` (``dims``, ``base``,
      ``scaling``: YaRN ``factor`` / ``original`` / ``fast`` / ``slow`` or absent), ``scale``,
      ``mask.size`` (sliding window) and optionally ``kv_from``: the layer has no K/V projections and
      reads that earlier layer's cached K/V with its own queries and window.
  rglru mixer: ``width`` (channels of the two branches), ``conv`` (taps), ``blocks`` (the gates are
      block-diagonal over that many equal channel groups).

Checkpoint tensor names: ``embed``, ``final.norm``, ``head``, and per layer ``l<i>.``: ``norm1``,
``norm1b``, ``norm2``, ``norm2b``; ``mix.q|k|v`` (+ ``.conv``, ``mix.q.norm``, ``mix.k.norm``), ``mix.o``;
``mix.y`` / ``mix.x`` (+ ``.b``), ``mix.conv`` (+ ``.b``), ``mix.ra`` / ``mix.ri`` [blocks, out, in] (+ ``.b``),
``mix.lam``; ``mlp.gate`` / ``mlp.up`` / ``mlp.down`` (+ ``.b``).  Linear weights are [out, in].

What a sequence keeps between steps: paged K/V of the attention layers that own projections (one block
table for all of them, from the engine's BlockManager) and one STATE SLOT (BlockManager state slots):
per layer the last ``conv - 1`` projected rows its convolution still needs, and per RG-LRU layer the
float32 recurrent state.  The stage runs the same interface as :class:`~.stage.ModelStage`
(``forward(ids, BatchMeta)``, ``allocate_kv``), so the engine, scheduler and sampler drive it
unchanged; it owns every layer (no pipeline cuts, no tensor parallelism).
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional

import torch

from .. import ops
from ..config import ModelConfig
from ..ops import seqmix as sm
from .stage import BatchMeta
from .weights import tensor_seed


# ----------------------------------------------------------------------------- sizes
def kv_width(layer: Dict[str, Any]) -> int:
    """K + V elements a token adds to the cache for this layer (0: no cache of its own)."""
    m = layer["mixer"]
    if layer["type"] != "attention" or "kv_from" in m:
        return 0
    return m["kv_heads"] * (m["dim"] + m["vdim"])


def layer_param_count(width: int, layer: Dict[str, Any]) -> int:
    return sum(int(torch.Size(s).numel()) for s in layer_shapes(width, layer).values())


def layer_shapes(width: int, layer: Dict[str, Any]) -> Dict[str, tuple]:
    """Checkpoint tensor name (without the ``l<i>.`` prefix) -> shape."""
    m = layer["mixer"]
    s: Dict[str, tuple] = {"norm1": (width,), "norm1b": (width,)}
    if layer["type"] == "attention":
        h, g, d, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        s.update({"mix.q": (h * d, width), "mix.q.norm": (d,), "mix.q.conv": (h * d, taps), "mix.o": (width, h * dv)})
        if "kv_from" not in m:
            s.update({"mix.k": (g * d, width), "mix.k.norm": (d,), "mix.k.conv": (g * d, taps),
                      "mix.v": (g * dv, width), "mix.v.conv": (g * dv, taps)})
    else:
        c, nb, taps = m["width"], m["blocks"], m["conv"]
        bw = c // nb
        s.update({"mix.y": (c, width), "mix.y.b": (c,), "mix.x": (c, width), "mix.x.b": (c,),
                  "mix.conv": (c, taps), "mix.conv.b": (c,), "mix.ra": (nb, bw, bw), "mix.ra.b": (nb, bw),
                  "mix.ri": (nb, bw, bw), "mix.ri.b": (nb, bw), "mix.lam": (c,), "mix.o": (width, c)})
    if layer.get("mlp"):
        f = layer["mlp"]["ff"]
        s.update({"norm2": (width,), "norm2b": (width,), "mlp.gate": (f, width), "mlp.gate.b": (f,),
                  "mlp.up": (f, width), "mlp.up.b": (f,), "mlp.down": (width, f), "mlp.down.b": (width,)})
    return s


def model_shapes(cfg: ModelConfig) -> Dict[str, tuple]:
    s = {"embed": (cfg.vocab_size, cfg.hidden_size), "final.norm": (cfg.hidden_size,),
         "head": (cfg.vocab_size, cfg.hidden_size)}
    for i, layer in enumerate(cfg.layers):
        s.update({f"l{i}.{n}": shp for n, shp in layer_shapes(cfg.hidden_size, layer).items()})
    return s


def synth_state_dict(cfg: ModelConfig, seed: int = 0, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Seeded random weights under the checkpoint names (CPU): projections ~ N(0, 1 / fan_in), norm
    weights and biases small around zero, ``lam`` spread so that decays differ per channel."""
    sd = {}
    for name, shape in model_shapes(cfg).items():
        g = torch.Generator().manual_seed(tensor_seed(seed, 0, name))
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        if leaf.endswith("lam"):
            t = torch.rand(shape, generator=g) * 4.0 - 3.0
        elif leaf in ("mix.q.norm", "mix.k.norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif len(shape) == 1 or leaf.endswith(".b"):
            t = 0.1 * torch.randn(shape, generator=g)
        elif leaf.endswith(".conv"):
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
        sd[name] = t.to(dtype)
    return sd


class LayerListStage:
    """What the stages of layer-list models share: one stage owns every layer of the ``config.json`` list
    on one device (no pipeline cuts, no tensor parallelism), a float32 residual stream, per-cache paged
    K/V tensors of their own shapes behind ONE block table (the engine's BlockManager), and the same
    interface as :class:`~.stage.ModelStage` (``forward(ids, BatchMeta)``, ``allocate_kv``,
    ``load_hf_state``, ``init_synthetic``), so the engine, scheduler and sampler drive them unchanged.
    A subclass gives ``cache_shapes`` (per cache key the K and V shapes inside a block), the weights
    and ``forward``."""

    def __init__(self, cfg: ModelConfig, layer_start: int = 0, layer_end: Optional[int] = None, device="cpu",
                 dtype=torch.bfloat16, units: Optional[tuple] = None, tp=None, unit_group: int = 2):
        from ..parallel.tensor_parallel import TPGroup
        if cfg.layers is None:
            raise ValueError(f"{type(self).__name__} needs a layer-list config")
        layer_end = cfg.num_layers if layer_end is None else layer_end
        if (layer_start, layer_end) != (0, cfg.num_layers) or (units is not None and tuple(units) != (
                0, unit_group * cfg.num_layers)):
            raise ValueError("a layer-list model runs as one stage (no pipeline cuts)")
        if tp is not None and tp.enabled:
            raise ValueError("a layer-list model runs without tensor parallelism")
        if dtype not in sm.ACT_DTYPES:
            raise ValueError(f"layer-list models run in bfloat16 or float32, not {dtype}")
        self.tp = tp if tp is not None else TPGroup(0, 1)
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.layer_start, self.layer_end = 0, cfg.num_layers
        self.is_first = self.is_last = True
        self.specs = cfg.layers
        self.hkv = cfg.num_kv_heads
        self.layers: List[Dict[str, torch.Tensor]] = []
        self.embed: Dict[str, torch.Tensor] = {}
        self.head: Dict[str, torch.Tensor] = {}
        self.kv = None                 # _PagedCaches: {cache key: (k_cache, v_cache)} + block_size / num_blocks
        self.state = None
        self.num_state_slots = 0
        self.taps = None               # optional list: the residual stream after every layer run (debugging)

    # ------------------------------------------------------------------ what a subclass provides
    def cache_shapes(self, block_size: int) -> Dict[Any, tuple]:
        """{cache key: (k shape, v shape)} of one block (without the leading block axis)."""
        raise NotImplementedError

    def quantize(self, mode):
        if mode not in ("", "none", None):
            raise ValueError("layer-list models run unquantized")
        return self

    def weight_bytes(self) -> int:
        def walk(o):
            if isinstance(o, torch.Tensor):
                return o.numel() * o.element_size()
            if isinstance(o, dict):
                return sum(walk(v) for v in o.values())
            return 0
        return sum(walk(d) for d in self.layers) + walk(self.embed) + walk(self.head)

    def lm_head_weight(self, full: bool = False) -> torch.Tensor:
        return self.head["lm_head"]

    def needs_embed(self) -> bool:
        return True

    @property
    def num_layers(self) -> int:
        """Caches that take a share of every block (what the K/V pool is planned for)."""
        return len(self.cache_shapes(1))

    # ------------------------------------------------------------------ cache
    def kv_bytes_per_block(self, block_size: int) -> int:
        e = torch.empty((), dtype=self.dtype).element_size()
        n = sum(torch.Size(k).numel() + torch.Size(v).numel() for k, v in self.cache_shapes(block_size).values())
        return max(1, n * e)

    def allocate_kv(self, num_blocks: int, block_size: int):
        caches = {key: (torch.zeros(num_blocks, *ks, dtype=self.dtype, device=self.device),
                        torch.zeros(num_blocks, *vs, dtype=self.dtype, device=self.device))
                  for key, (ks, vs) in self.cache_shapes(block_size).items()}
        self.kv = _PagedCaches(caches, num_blocks, block_size)
        return self.kv

    def _seq_batch(self, meta: BatchMeta) -> sm.SeqBatch:
        if meta.tok_seq is None or meta.cu_seqlens_q is None or (
                self.cfg.needs_state_slots and meta.state_slots is None):
            raise RuntimeError("a layer-list model needs varlen metadata in every step (and, with per-sequence "
                               "state, a BlockManager with num_state_slots > 0)")
        return sm.SeqBatch(meta.cu_seqlens_q, meta.positions, meta.tok_seq, meta.state_slots, meta.num_seqs,
                           meta.num_tokens, max(1, meta.max_q_len))


class HybridStage(LayerListStage):
    """All layers of a Tudilix model on one device (see the module docstring)."""

    @staticmethod
    def layer_param_count(width: int, layer: Dict[str, Any]) -> int:
        return layer_param_count(width, layer)

    @staticmethod
    def kv_elements_per_token(cfg: ModelConfig) -> int:
        return sum(kv_width(l) for l in cfg.layers)

    def __init__(self, cfg: ModelConfig, layer_start: int = 0, layer_end: Optional[int] = None, device="cpu",
                 dtype=torch.bfloat16, units: Optional[tuple] = None, tp=None, unit_group: int = 2):
        super().__init__(cfg, layer_start, layer_end, device, dtype, units, tp, unit_group)
        for i, layer in enumerate(self.specs):
            m = layer["mixer"]
            if layer["type"] == "attention":
                if m["heads"] % m["kv_heads"] or m["rot"]["dims"] % 2 or m["rot"]["dims"] > m["dim"]:
                    raise ValueError(f"layer {i}: heads / kv_heads / rot.dims do not fit")
                j = m.get("kv_from")
                if j is not None:
                    src = self.specs[j]
                    if not (0 <= j < i) or src["type"] != "attention" or "kv_from" in src["mixer"]:
                        raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with K/V of its own")
                    if any(src["mixer"][k] != m[k] for k in ("kv_heads", "dim", "vdim")):
                        raise ValueError(f"layer {i}: kv_from layer has other K/V sizes")
            elif m["width"] % m["blocks"]:
                raise ValueError(f"layer {i}: width is not a multiple of blocks")
        self.kv_layers = [i for i, l in enumerate(self.specs) if kv_width(l)]
        self.state = None              # per layer {"conv": ..., "s": ...}
        self.rot = {}                  # layer -> (freqs [dims/2] f32, magnitude)
        for i, l in enumerate(self.specs):
            if l["type"] == "attention":
                r = l["mixer"]["rot"]
                f, mag = sm.yarn_frequencies(r["dims"], r["base"], r.get("scaling"))
                self.rot[i] = (f.to(self.device), mag)

    # ------------------------------------------------------------------ weights
    def load_hf_state(self, sd: Dict[str, torch.Tensor]) -> "HybridStage":
        """From checkpoint-named tensors: fuses y|x, q|k|v (and their convolutions), gate|up, and stores
        the gate matrices transposed ([blocks, in, out]) and the convolution weights tap-major ([taps, C])."""
        want = model_shapes(self.cfg)
        for n, shp in want.items():
            if n not in sd:
                raise KeyError(f"checkpoint lacks {n}")
            if tuple(sd[n].shape) != tuple(shp):
                raise ValueError(f"{n}: shape {tuple(sd[n].shape)}, config says {tuple(shp)}")
        cv = lambda t: t.to(device=self.device, dtype=self.dtype).contiguous()
        cat = lambda names: cv(torch.cat([sd[n] for n in names], 0))
        self.embed = {"embed": cv(sd["embed"])}
        self.head = {"final_norm": cv(sd["final.norm"]), "lm_head": cv(sd["head"])}
        self.layers = []
        for i, layer in enumerate(self.specs):
            p = f"l{i}."
            w = {k: cv(sd[p + k]) for k in ("norm1", "norm1b")}
            if layer["type"] == "attention":
                parts = ["q"] if "kv_from" in layer["mixer"] else ["q", "k", "v"]
                w["wqkv"] = cat([p + f"mix.{x}" for x in parts])
                w["conv_w"] = cv(torch.cat([sd[p + f"mix.{x}.conv"] for x in parts], 0).t())     # [taps, C]
                w["q_norm"] = cv(sd[p + "mix.q.norm"])
                if len(parts) == 3:
                    w["k_norm"] = cv(sd[p + "mix.k.norm"])
            else:
                w["w_yx"] = cat([p + "mix.y", p + "mix.x"])
                w["conv_w"] = cv(sd[p + "mix.conv"].t())                                        # [taps, C]
                for k, n in (("y_b", "mix.y.b"), ("x_b", "mix.x.b"), ("conv_b", "mix.conv.b"),
                             ("ra_b", "mix.ra.b"), ("ri_b", "mix.ri.b"), ("lam", "mix.lam")):
                    w[k] = cv(sd[p + n])
                w["ra_t"] = cv(sd[p + "mix.ra"].transpose(1, 2))
                w["ri_t"] = cv(sd[p + "mix.ri"].transpose(1, 2))
            w["wo"] = cv(sd[p + "mix.o"])
            if layer.get("mlp"):
                w["norm2"], w["norm2b"] = cv(sd[p + "norm2"]), cv(sd[p + "norm2b"])
                w["w_gu"] = cat([p + "mlp.gate", p + "mlp.up"])
                w["b_gu"] = cat([p + "mlp.gate.b", p + "mlp.up.b"])
                w["w_down"], w["b_down"] = cv(sd[p + "mlp.down"]), cv(sd[p + "mlp.down.b"])
            self.layers.append(w)
        return self

    def init_synthetic(self, seed: int = 0) -> "HybridStage":
        return self.load_hf_state(synth_state_dict(self.cfg, seed))

    # ------------------------------------------------------------------ cache and state
    def cache_shapes(self, block_size: int) -> Dict[Any, tuple]:
        """Paged caches of the attention layers with K/V of their own: k [NB, G, BS, dim],
        v [NB, G, vdim, BS] (transposed inside a block); a ``kv_from`` layer reads its source's pair."""
        out = {}
        for i in self.kv_layers:
            m = self.specs[i]["mixer"]
            out[i] = ((m["kv_heads"], block_size, m["dim"]), (m["kv_heads"], m["vdim"], block_size))
        return out

    def allocate_state(self, num_slots: int):
        """State pools, one row per BlockManager state slot: per layer the convolution tail
        [slots, taps - 1, C] (activation dtype) and per RG-LRU layer the state [slots, C] float32."""
        self.num_state_slots = num_slots
        self.state = []
        for l in self.specs:
            m = l["mixer"]
            if l["type"] == "attention":
                c = m["heads"] * m["dim"] + (0 if "kv_from" in m else m["kv_heads"] * (m["dim"] + m["vdim"]))
                st = {}
            else:
                c = m["width"]
                st = {"s": torch.zeros(num_slots, c, dtype=torch.float32, device=self.device)}
            st["conv"] = torch.zeros(num_slots, max(0, m["conv"] - 1), c, dtype=self.dtype, device=self.device)
            self.state.append(st)
        return self.state

    def state_bytes_per_slot(self) -> int:
        e = torch.empty((), dtype=self.dtype).element_size()
        n = 0
        for l in self.specs:
            m = l["mixer"]
            if l["type"] == "attention":
                c = m["heads"] * m["dim"] + (0 if "kv_from" in m else m["kv_heads"] * (m["dim"] + m["vdim"]))
            else:
                c = m["width"]
                n += 4 * c
            n += e * c * (m["conv"] - 1)
        return n

    # ------------------------------------------------------------------ forward
    def _attention(self, i: int, h: torch.Tensor, w, meta: BatchMeta, sb: sm.SeqBatch) -> torch.Tensor:
        m = self.specs[i]["mixer"]
        own = "kv_from" not in m
        kc, vc = self.kv.caches[i if own else m["kv_from"]]
        freqs, mag = self.rot[i]
        qkv = ops.linear(h, w["wqkv"])
        q = sm.attn_prep(qkv, w["conv_w"], self.state[i]["conv"], w["q_norm"], w.get("k_norm"), freqs, mag,
                         self.cfg.norm_eps, kc if own else None, vc if own else None, meta.slot_mapping, sb,
                         m["heads"], m["kv_heads"], m["dim"], m["vdim"])
        nd = meta.num_decode if meta.is_prefill else meta.num_seqs
        window = int((m.get("mask") or {}).get("size") or (1 << 30))          # no mask entry: plain causal attention
        scale = float(m["scale"]) if m.get("scale") is not None else m["dim"] ** -0.5
        a = sm.window_attention(q, kc, vc, meta.block_tables, sb, window, scale, num_decode=nd)
        return ops.linear(a.view(a.shape[0], -1), w["wo"])

    def _rglru(self, i: int, h: torch.Tensor, w, sb: sm.SeqBatch) -> torch.Tensor:
        m = self.specs[i]["mixer"]
        c = m["width"]
        yx = ops.linear(h, w["w_yx"])
        st = self.state[i]
        u = sm.causal_conv(yx[:, c:], w["conv_w"], w["conv_b"], st["conv"], sb, in_bias=w["x_b"])
        r = sm.rglru(u, yx[:, :c], w["y_b"], w["ra_t"], w["ra_b"], w["ri_t"], w["ri_b"], w["lam"], st["s"], sb,
                     self.dtype)
        return ops.linear(r, w["wo"])

    @torch.inference_mode()
    def forward(self, inp: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        if self.kv is None or self.state is None:
            raise RuntimeError("allocate_kv() and allocate_state() before forward()")
        cfg = self.cfg
        eps, mult = cfg.norm_eps, cfg.residual_mult
        sb = self._seq_batch(meta)
        x = sm.embedding_f32(inp, self.embed["embed"])
        h = sm.rms_norm_f32(x, self.layers[0]["norm1"], eps, self.dtype)
        n = len(self.layers)
        for i, (spec, w) in enumerate(zip(self.specs, self.layers)):
            o = self._attention(i, h, w, meta, sb) if spec["type"] == "attention" else self._rglru(i, h, w, sb)
            nxt = self.layers[i + 1]["norm1"] if i + 1 < n else None
            x, h = sm.post_norm_add(x, o, w["norm1b"], eps, mult, w_next=w["norm2"] if spec.get("mlp") else nxt)
            if spec.get("mlp"):
                y = sm.clipped_glu(ops.linear(h, w["w_gu"]), w["b_gu"], spec["mlp"]["limit"])
                x, h = sm.post_norm_add(x, ops.linear(y, w["w_down"]), w["norm2b"], eps, mult, bias=w["b_down"],
                                        w_next=nxt)
            if self.taps is not None:
                self.taps.append(x.clone())
        if meta.logits_idx is not None:
            x = x.index_select(0, meta.logits_idx)
        hf = sm.rms_norm_f32(x, self.head["final_norm"], eps, self.dtype)
        return sm.softcap_f32(ops.linear(hf, self.head["lm_head"]), cfg.logit_softcap)


class _PagedCaches:
    """Per-layer paged K/V tensors of a :class:`HybridStage` (the role of stage.KVCache)."""

    def __init__(self, caches, num_blocks: int, block_size: int):
        self.caches, self.num_blocks, self.block_size = caches, num_blocks, block_size

    @property
    def nbytes(self) -> int:
        return sum(k.numel() * k.element_size() + v.numel() * v.element_size() for k, v in self.caches.values())
