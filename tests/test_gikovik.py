"""The Gikovik decoder (latent attention with a sink or a shared rotated key part, parallel layers,
grouped-choice mixture of experts, per-layer token input, a looped span of layers) against the plain
float64 oracle of tests/oracle_gikovik.py: every mechanism alone, then the engine -- whole prompts,
token-by-token decoding, prompt portions down to two tokens, batches of unequal requests, blocks that
are freed and used again, keys far away and at block borders, the first tokens, long decoding, and
greedy generation through the scheduler.  Each case runs on the CPU path in float32 and, marked gpu,
on the HIP kernels in float32 and bfloat16.
"""
import json

import numpy as np
import pytest
import torch

import oracle_gikovik as O
from distributed_llms_amd.config import EngineConfig, ModelConfig
from distributed_llms_amd.engine.llm_engine import LLMEngine
from distributed_llms_amd.engine.replay import TraceReplayer
from distributed_llms_amd.engine.sequence import SamplingParams
from distributed_llms_amd.models import make_stage
from distributed_llms_amd.ops import latent as lat
from distributed_llms_amd.ops import moe
from distributed_llms_amd.ops import seqmix as sm

gpu = pytest.mark.gpu
TARGETS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
           pytest.param(("cuda", torch.float32), id="gpu-f32", marks=gpu),
           pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=gpu)]


def _rot_mixer(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base=10000.0, dims=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
            "scale": scale, "rot": {"base": base, "dims": rot_dim if dims is None else dims}}


def _sink_mixer(heads, dim, vdim, kv_rank, q_rank, scale):
    return {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale}


def _moe(experts, count, keep, top, scale, ff, shared):
    return {"kind": "moe", "expert": {"ff": ff}, "shared": {"ff": shared} if shared else None,
            "router": {"experts": experts, "groups": {"count": count, "keep": keep}, "scale": scale, "top": top}}


def cfg_a():
    """A loop over the two middle layers (not from layer 0, not to the end), both mixers with different
    shapes per layer, key widths on both sides of the kernels' tiles, experts in groups with fewer kept
    than there are, a shared expert of another size than the experts, a layer without feed-forward."""
    return {"architecture": "Gikovik", "vocab": 200, "width": 96, "norm": {"eps": 1e-6}, "token_side": {"dim": 8},
            "loop": {"start": 1, "stop": 3, "times": 2},
            "layers": [
                {"type": "latent_attention_2", "mixer": _rot_mixer(4, 24, 8, 40, 48, 56, 0.2),
                 "mlp": {"kind": "dense", "ff": 160}},
                {"type": "latent_attention", "mixer": _sink_mixer(6, 16, 24, 32, 40, 0.25),
                 "mlp": _moe(8, 4, 2, 3, 2.0, 48, 40)},
                {"type": "latent_attention_2", "mixer": _rot_mixer(2, 32, 16, 16, 40, 24, 0.3, base=500.0),
                 "mlp": _moe(6, 3, 3, 2, 1.0, 32, 0)},
                {"type": "latent_attention", "mixer": _sink_mixer(3, 8, 12, 20, 16, 0.4), "mlp": None},
            ]}


def cfg_b():
    """Degenerate sizes: one head, one expert per token, one group, groups of one expert, a two-column
    token input (one column is checked with the mechanism alone: it is ill-conditioned where its gate is near zero), a loop of one layer that runs three times, no shared expert, odd widths."""
    return {"architecture": "Gikovik", "vocab": 131, "width": 72, "norm": {"eps": 1e-5}, "token_side": {"dim": 2},
            "loop": {"start": 2, "stop": 3, "times": 3},
            "layers": [
                {"type": "latent_attention", "mixer": _sink_mixer(1, 12, 20, 12, 12, 0.3), "mlp": _moe(2, 1, 1, 1, 1.0, 24, 0)},
                {"type": "latent_attention_2", "mixer": _rot_mixer(1, 10, 6, 14, 18, 22, 0.25, dims=4),
                 "mlp": _moe(4, 4, 2, 2, 0.5, 16, 8)},
                {"type": "latent_attention_2", "mixer": _rot_mixer(5, 8, 2, 8, 8, 8, 0.35, base=100.0),
                 "mlp": {"kind": "dense", "ff": 40}},
            ]}


def cfg_c():
    """No loop and no token input at all; expert sizes that the grouped GPU kernels take."""
    return {"architecture": "Gikovik", "vocab": 160, "width": 128, "norm": {"eps": 1e-6},
            "layers": [
                {"type": "latent_attention_2", "mixer": _rot_mixer(4, 32, 16, 32, 64, 64, 0.15),
                 "mlp": _moe(8, 2, 1, 2, 1.5, 128, 64)},
                {"type": "latent_attention", "mixer": _sink_mixer(2, 32, 48, 64, 32, 0.2),
                 "mlp": {"kind": "dense", "ff": 256}},
            ]}


CONFIGS = {"a": cfg_a, "b": cfg_b, "c": cfg_c}


def _round(sd, dtype):
    """Weights as the engine will hold them (rounded to bf16 for a bf16 run), for engine and oracle."""
    return {k: torch.from_numpy(v).to(dtype).float() for k, v in sd.items()}


def make_engine(cfg, sd, target, tmp_path, max_tokens=512, max_requests=4, block_size=32, graphs=False):
    device, dtype = target
    if device == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    mcfg = ModelConfig.from_hf_config(cfg)
    stage = make_stage(mcfg, device=device, dtype=dtype).load_hf_state(sd)
    ecfg = EngineConfig(model=str(tmp_path), shard_dir=str(tmp_path), device=device,
                        dtype="float32" if dtype == torch.float32 else "bfloat16", max_batch=max_requests,
                        max_seq_len=max_tokens + 1, kv_block_size=block_size,
                        num_kv_blocks=-(-max_tokens // block_size) + max_requests + 1,
                        max_prefill_tokens=max_tokens, use_graphs=graphs, graph_batch_sizes=(1, 2, 4))
    return LLMEngine(ecfg, stage)


def row_errs(got, want):
    """Per position: rms of the difference (mean over the vocabulary taken off) over the rms of the oracle's logits."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((want ** 2).mean())


def oracle(cfg, sd, tokens, taps=None):
    """(logits, decided): ``decided`` [T] marks the positions up to which no token's expert choice was a
    close call in any layer run (the choice of a token also reaches later positions, through attention)."""
    margins = []
    want = O.forward(cfg, sd, np.array(tokens), taps, margins)
    ok = np.ones(len(tokens), dtype=bool)
    for m in margins:
        ok &= m > 0.1
    return want, np.logical_and.accumulate(ok)


def assert_close(got, want, target, what="", bf16_slack=1.0):
    """``want``: (logits, decided) of :func:`oracle`.  float32: positions within 1e-5 at the median and
    5e-4 at most (where a token-input gate is near zero the norm behind it amplifies float32 rounding a
    hundredfold; a wrong key, weight or state shows at 1e-2 and more).  bfloat16: within 4e-2 at every
    position before the first close call of a router (rounded activations may turn it the other way,
    which is no fault), 2e-2 at their median; ``bf16_slack`` widens both for the model of degenerate sizes,
    whose 8- to 12-wide latents and thrice-run layer make every bfloat16 rounding count for more."""
    want, decided = want
    e = row_errs(got, want)
    if target[1] == torch.float32:
        assert np.median(e) < 1e-5 and e.max() < 5e-4, (what, float(np.median(e)), float(e.max()), int(e.argmax()))
    elif decided.any():
        d = e[decided]
        assert np.median(d) < 2e-2 * bf16_slack and d.max() < 4e-2 * bf16_slack, (
            what, int(decided.sum()), float(np.median(d)), float(d.max()))


def replay(engine, schedule, prompts):
    """schedule: steps, each a list of (request name, token count); returns name -> logits [len, V]."""
    rp = TraceReplayer(engine)
    at = {n: 0 for n in prompts}
    out = {n: [] for n in prompts}
    for step in schedule:
        entries, end = [], []
        for n, c in step:
            toks = prompts[n][at[n]:at[n] + c]
            entries.append((n, toks, list(range(len(toks)))))
            at[n] += c
            if at[n] == len(prompts[n]):
                end.append(n)
        logits = rp.step(entries, end).cpu().numpy()
        row = 0
        for n, toks, _ in entries:
            out[n].append(logits[row:row + len(toks)])
            row += len(toks)
    return {n: np.concatenate(v) for n, v in out.items() if v}


def prompts_for(cfg, lens, seed=1):
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, cfg["vocab"], n).tolist() for i, n in enumerate(lens)}


def _sb(chunks, device):
    """SeqBatch for chunks [(start position, length)]."""
    cu = np.concatenate([[0], np.cumsum([n for _, n in chunks])]).astype(np.int32)
    pos = np.concatenate([np.arange(s, s + n) for s, n in chunks]).astype(np.int32)
    seq = np.concatenate([np.full(n, i) for i, (_, n) in enumerate(chunks)]).astype(np.int32)
    t = lambda a: torch.from_numpy(a).to(device)
    return sm.SeqBatch(t(cu), t(pos), t(seq), None, len(chunks), int(cu[-1]), max(n for _, n in chunks))


def _dev(target):
    if target[0] == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return target


def _atol(dtype, f32=2e-5, bf16=3e-2):
    return f32 if dtype == torch.float32 else bf16


# ------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [(4, 56, 48, 16), (6, 32, 32, 32), (3, 20, 20, 16), (2, 192, 160, 32), (20, 40, 40, 32)])
def test_sink_and_far_keys_over_one_shared_head(target, shape):
    """Attention of H query heads over ONE shared K/V head, causal over the whole sequence.  (a) A sink
    far above every score leaves almost nothing of the output, one far below changes nothing, ordinary
    ones are the oracle's; (b) one key far back (among hundreds, on both sides of block borders, the
    very first one) gets a score far above the rest and owns the output -- as a prompt portion and for
    a decoded token, blocks scattered in the pool."""
    device, dtype = _dev(target)
    h, d, dv, bs = shape
    rng = np.random.default_rng(h * d)
    n = 300
    q = rng.standard_normal((n, h, d)).astype(np.float32) * 0.5
    k = rng.standard_normal((n, 1, d)).astype(np.float32) * 0.5
    v = rng.standard_normal((n, 1, dv)).astype(np.float32)
    table = list(rng.permutation(np.arange(1, 40))[:-(-n // bs)])
    T = lambda a: torch.from_numpy(a).to(dtype)

    def paged(kk, vv):
        kc = torch.zeros(40, 1, bs, d, dtype=dtype)
        vc = torch.zeros(40, 1, dv, bs, dtype=dtype)
        for j in range(n):
            kc[table[j // bs], :, j % bs] = kk[j]
            vc[table[j // bs], :, :, j % bs] = vv[j]
        return kc.to(device), vc.to(device)

    def oracle(qq, kk, vv, sinks):
        out = np.zeros((n, h, dv))
        for a in range(h):
            s = qq[:, a].double().numpy() @ kk[:, 0].double().numpy().T * 0.3
            out[:, a] = O.causal_softmax_mix(s, vv[:, 0].double().numpy(), None if sinks is None else float(sinks[a]))
        return out

    bt = torch.tensor([table], dtype=torch.int32, device=device)
    tol = _atol(dtype)

    def both(qq, kc, vc, sinks, want, p, span=12):
        st = None if sinks is None else torch.tensor(sinks, dtype=torch.float32, device=device)
        lo = max(0, p - span + 1)
        o = sm.window_attention(qq[lo:p + 1].contiguous().to(device), kc, vc, bt, _sb([(lo, p + 1 - lo)], device),
                                1 << 30, 0.3, num_decode=0, sinks=st)
        np.testing.assert_allclose(o.float().cpu().numpy(), want[lo:p + 1], rtol=tol, atol=tol)
        o = sm.window_attention(qq[p:p + 1].contiguous().to(device), kc, vc, bt, _sb([(p, 1)], device), 1 << 30, 0.3,
                                sinks=st)
        np.testing.assert_allclose(o.float().cpu().numpy(), want[p:p + 1], rtol=tol, atol=tol)

    qq, kk, vv = T(q), T(k), T(v)
    kc, vc = paged(kk, vv)
    plain = oracle(qq, kk, vv, None)
    for sinks in (list(rng.standard_normal(h) * 1.5), [30.0] * h, [-40.0] * h):
        want = oracle(qq, kk, vv, sinks)
        for p in (0, 1, 70, n - 1):
            both(qq, kc, vc, sinks, want, p)
        if sinks[0] == 30.0:
            assert np.abs(want[5:]).max() < 1e-6 * np.abs(plain).max() + 1e-6        # the test bites
        if sinks[0] == -40.0:
            np.testing.assert_allclose(want, plain, atol=1e-12)
    # whole sequence in one portion, with ordinary sinks
    sinks = list(rng.standard_normal(h))
    st = torch.tensor(sinks, dtype=torch.float32, device=device)
    o = sm.window_attention(qq.to(device), kc, vc, bt, _sb([(0, n)], device), 1 << 30, 0.3, num_decode=0, sinks=st)
    np.testing.assert_allclose(o.float().cpu().numpy(), oracle(qq, kk, vv, sinks), rtol=tol, atol=tol)
    # (b) a far key
    for p, j in ((n - 1, 0), (n - 1, bs - 1), (n - 1, bs), (n - 1, 2 * bs + 1), (200, 3), (bs, bs - 1), (bs, bs)):
        k2, q2 = k.copy(), q.copy()
        k2[j] = 0.0
        k2[j, :, 0] = 8.0
        q2[p, :, 0] = 16.0                  # score 16 * 8 * 0.3 far above the rest
        qq, kk = T(q2), T(k2)
        kc, vc = paged(kk, vv)
        want = oracle(qq, kk, vv, None)
        np.testing.assert_allclose(want[p, 0], vv[j, 0].double().numpy(), atol=1e-3)
        both(qq, kc, vc, None, want, p, span=5)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [(4, 56, 48), (20, 192, 160)])
def test_decode_rows_with_their_keys_cut_into_runs(target, shape, monkeypatch):
    """Few decode rows of long context: each row's keys are cut into runs on separate workgroups and
    the partial softmaxes merged (with the sink).  Rows of different lengths in one batch -- one so
    short that most runs are empty -- equal the oracle, whatever the number of runs."""
    device, dtype = _dev(target)
    h, d, dv = shape
    bs, lens = 32, [700, 33, 257]
    rng = np.random.default_rng(h)
    T = lambda a: torch.from_numpy(a.astype(np.float32)).to(dtype)
    nb = sum(-(-n // bs) for n in lens) + 1
    kc = torch.zeros(nb, 1, bs, d, dtype=dtype)
    vc = torch.zeros(nb, 1, dv, bs, dtype=dtype)
    sinks = list(rng.standard_normal(h))
    tables, qs, wants, blk = [], [], [], 1
    for n in lens:
        k, v = T(rng.standard_normal((n, d)) * 0.5), T(rng.standard_normal((n, dv)))
        q = T(rng.standard_normal((h, d)) * 0.5)
        table = list(range(blk, blk + -(-n // bs)))
        blk += len(table)
        for j in range(n):
            kc[table[j // bs], 0, j % bs] = k[j]
            vc[table[j // bs], 0, :, j % bs] = v[j]
        s = q.double().numpy() @ k.double().numpy().T * 0.3                      # [h, n]
        want = np.zeros((h, dv))
        for a in range(h):
            row = np.full((n, n), -1e30)
            row[n - 1] = s[a]
            want[a] = O.causal_softmax_mix(row, v.double().numpy(), float(sinks[a]))[n - 1]
        tables.append(table + [0] * (32 - len(table)))
        qs.append(q)
        wants.append(want)
    bt = torch.tensor(tables, dtype=torch.int32, device=device)
    q = torch.stack(qs).to(device)
    st = torch.tensor(sinks, dtype=torch.float32, device=device)
    cu = torch.arange(len(lens) + 1, dtype=torch.int32, device=device)
    pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32, device=device)
    sb = sm.SeqBatch(cu, pos, cu[:-1].contiguous(), None, len(lens), len(lens), 1)
    for min_keys in (256, 64, 32):
        monkeypatch.setattr(sm, "DECODE_SPLIT_KEYS", min_keys)
        assert sm.decode_splits(3, h, 1, 700) == min(700 // min_keys, 512 // (3 * -(-h // 16)), 64)
        o = sm.window_attention(q, kc.to(device), vc.to(device), bt, sb, 1 << 30, 0.3, sinks=st, max_ctx=700)
        np.testing.assert_allclose(o.float().cpu().numpy(), np.stack(wants), rtol=_atol(dtype), atol=_atol(dtype))


def _mixer_weights(layer, width, seed, dtype):
    cfg = {"vocab": 4, "width": width, "norm": {"eps": 1e-6}, "layers": [layer]}
    sd = O.make_weights(cfg, seed)
    return {k[len("l0.mix."):]: torch.from_numpy(v).to(dtype).float().numpy() for k, v in sd.items()
            if k.startswith("l0.mix.")}


def _stage_mixer(p, layer, dtype, device):
    """The mixer's weights in the layout ops.latent takes (as the stage's loader makes them)."""
    from distributed_llms_amd.models.gikovik import latent_spec
    sp = latent_spec(layer)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device=device, dtype=dtype).contiguous()
    parts = [p["dq"], p["dkv"]] + ([p["g"]] if sp.gated else [])
    w = {"down": t(np.concatenate(parts, 0)), "q_norm": t(p["dq.norm"]), "c_norm": t(p["dkv.norm"]), "uq": t(p["uq"]),
         "uk": t(p["uk"].reshape(sp.heads, sp.dim, sp.rank)),
         "uv_t": t(p["uv"].reshape(sp.heads, sp.vdim, sp.rank).transpose(0, 2, 1)), "o": t(p["o"])}
    if not sp.gated:
        w["sinks"] = torch.from_numpy(p["sink"]).float().to(device)
    return sp, w


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("layer", [
    {"type": "latent_attention", "mixer": _sink_mixer(4, 16, 24, 32, 40, 0.3)},
    {"type": "latent_attention", "mixer": _sink_mixer(1, 9, 5, 7, 11, 0.5)},
    {"type": "latent_attention_2", "mixer": _rot_mixer(4, 24, 8, 40, 48, 56, 0.2)},
    {"type": "latent_attention_2", "mixer": _rot_mixer(3, 16, 12, 16, 20, 16, 0.25, base=50.0, dims=8)},
    {"type": "latent_attention_2", "mixer": _rot_mixer(18, 16, 16, 8, 112, 32, 0.2)},
], ids=["sink", "sink-odd", "rot", "rot-partial", "rot-18heads"])
def test_latent_mixers_through_the_cache(target, layer):
    """Each mixer alone over a paged latent cache: a whole sequence at once, then the same in portions
    (cut inside blocks, down to two tokens) and single tokens, equal to the oracle that computes keys
    and values per head from the latent."""
    device, dtype = _dev(target)
    width, n, bs = 64, 75, 16
    p = _mixer_weights(layer, width, 5, dtype)
    sp, w = _stage_mixer(p, layer, dtype, device)
    rng = np.random.default_rng(2)
    h = torch.from_numpy(rng.standard_normal((n, width)).astype(np.float32)).to(dtype)
    fn = O.latent_attention_sink if layer["type"] == "latent_attention" else O.latent_attention_rot
    want = fn(h.double().numpy(), {k: v.astype(np.float64) for k, v in p.items()}, layer["mixer"], 1e-6)
    freqs = None
    if sp.rot_dim:
        r = layer["mixer"]["rot"]
        freqs = sm.yarn_frequencies(r["dims"], r["base"], None)[0].to(device)
    table = [7, 2, 9, 4, 1]
    bt = torch.tensor([table], dtype=torch.int32, device=device)
    scale = np.abs(want).max()
    for sizes in ([n], [2, 14, 1, 17, 3, 1, 1, 30, 2, 4]):
        assert sum(sizes) == n
        kc = torch.zeros(10, 1, bs, sp.key_width, dtype=dtype, device=device)
        vc = torch.zeros(10, 1, sp.rank, bs, dtype=dtype, device=device)
        got, at = [], 0
        for c in sizes:
            pos = np.arange(at, at + c)
            slots = torch.tensor([table[j // bs] * bs + j % bs for j in pos], dtype=torch.int32, device=device)
            sb = _sb([(at, c)], device)
            nd = 1 if c == 1 and at > 0 else 0
            got.append(lat.latent_attention(h[at:at + c].contiguous().to(device), w, sp, freqs, 1e-6, kc, vc, slots,
                                            bt, sb, num_decode=nd).float().cpu().numpy())
            at += c
        tol = _atol(dtype, 3e-5, 4e-2) * scale
        np.testing.assert_allclose(np.concatenate(got), want, rtol=0, atol=tol)


@pytest.mark.parametrize("target", TARGETS)
def test_rotation_far_positions(target):
    """The shared key part and the queries' rotated part at positions in the tens of thousands: angles
    are float32 products of the position and the frequency."""
    device, dtype = _dev(target)
    sp = lat.LatentSpec(heads=2, dim=4, vdim=4, rank=8, q_rank=8, scale=1.0, rot_dim=6)
    freqs = sm.yarn_frequencies(4, 10000.0, None)[0].to(device)          # 4 of the 6 dimensions turn
    rng = np.random.default_rng(0)
    pos = np.array([0, 1, 31, 4097, 60001], dtype=np.int32)
    n = len(pos)
    q = torch.from_numpy(rng.standard_normal((n, 2 * 10)).astype(np.float32)).to(dtype)
    uk = torch.from_numpy(rng.standard_normal((2, 4, 8)).astype(np.float32)).to(dtype)
    qf = lat.latent_queries(q.to(device), uk.to(device), sp, freqs, torch.from_numpy(pos).to(device)).float().cpu().numpy()
    q3 = q.double().numpy().reshape(n, 2, 10)
    for t in range(n):
        want = O.rotate_pairs(q3[t:t + 1, :, 4:], 10000.0, 4, first_pos=int(pos[t]))[0]
        ang_err = 4e-3 * pos[t] / 6e4 + 1e-5            # float32 angle: relative 6e-8 of up to 6e4 radians
        np.testing.assert_allclose(qf[t, :, 8:], want, atol=_atol(dtype, 2e-5, 3e-2) + 4 * ang_err)
        np.testing.assert_allclose(qf[t, :, :8], np.einsum("hd,hdr->hr", q3[t, :, :4], uk.double().numpy()),
                                   atol=_atol(dtype, 2e-5, 6e-2))


def _router_case(rng, n, e, width):
    return {"router": rng.standard_normal((e, width)) * 4.0 / np.sqrt(width),
            "correction": rng.standard_normal(e) * 0.5 - 0.6}, rng.standard_normal((n, width))


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("r", [
    {"experts": 8, "groups": {"count": 4, "keep": 2}, "top": 3, "scale": 2.5},
    {"experts": 8, "groups": {"count": 4, "keep": 3}, "top": 4, "scale": 1.0},
    {"experts": 6, "groups": {"count": 6, "keep": 3}, "top": 2, "scale": 0.5},      # groups of one expert
    {"experts": 5, "groups": {"count": 1, "keep": 1}, "top": 1, "scale": 1.0},
    {"experts": 40, "groups": {"count": 5, "keep": 2}, "top": 9, "scale": 1.0},
    {"experts": 12, "top": 12, "scale": 3.0},                                       # everything chosen, no groups
])
def test_router_choice_and_weights(target, r):
    """Chosen experts and weights against the oracle.  Corrections are mostly negative, so choice scores
    of both signs occur: an expert of a dropped group must lose against a kept one with a NEGATIVE
    selection value (a dropped expert is masked with -inf; masking with zero would let it win), and the
    weights are the scores without the correction."""
    device, dtype = _dev(target)
    rng = np.random.default_rng(r["experts"] * 7 + r["top"])
    p, h = _router_case(rng, 200, r["experts"], 32)
    chosen, weights = O.route(h, p, r)
    g = r.get("groups") or {"count": 1, "keep": 1}
    logits = torch.from_numpy(h @ p["router"].T).float().to(device)
    corr = torch.from_numpy(p["correction"]).float().to(device)
    tw, ids = moe.route_grouped_choice(logits, corr, r["experts"], r["top"], g["count"], g["keep"], r["scale"])
    for t in range(200):
        assert set(ids[t].tolist()) == set(chosen[t].tolist()), t
        order = np.argsort(ids[t].cpu().numpy())
        np.testing.assert_allclose(tw[t].cpu().numpy()[order], weights[t][np.argsort(chosen[t])], rtol=2e-5)
    if g["keep"] < g["count"]:
        s = O.sigmoid(h @ p["router"].T) + p["correction"]
        assert any(s[t, chosen[t]].min() < 0 for t in range(200))                       # the test bites


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("case", [(8, 4, 2, 3, 48, 40, 96, 70), (6, 3, 3, 2, 32, 0, 72, 33), (2, 1, 1, 1, 24, 0, 40, 5),
                                  (8, 2, 1, 2, 128, 64, 128, 40), (8, 4, 3, 4, 256, 256, 256, 300), (4, 4, 2, 2, 16, 8, 24, 1)])
def test_expert_feed_forward(target, case):
    """The whole mixture (router, squared-ReLU experts, weighted sum, gated shared expert) against the
    oracle, at sizes the grouped GPU kernels take (few and many tokens) and at sizes they do not."""
    device, dtype = _dev(target)
    e, count, keep, top, ff, shared, width, n = case
    mlp = _moe(e, count, keep, top, 1.7, ff, shared)
    rng = np.random.default_rng(e + n)
    rd = lambda a: torch.from_numpy(a.astype(np.float32)).to(dtype).double().numpy()
    p = {"router": rd(rng.standard_normal((e, width)) * 4.0 / np.sqrt(width)), "correction": rd(rng.standard_normal(e) * 0.4)}
    for j in range(e):
        p[f"e{j}.up"] = rd(rng.standard_normal((ff, width)) / np.sqrt(width))
        p[f"e{j}.down"] = rd(rng.standard_normal((width, ff)) / np.sqrt(ff))
    if shared:
        p.update({"shared.up": rd(rng.standard_normal((shared, width)) / np.sqrt(width)),
                  "shared.down": rd(rng.standard_normal((width, shared)) / np.sqrt(shared)),
                  "shared.sg": rd(rng.standard_normal((1, width)) / np.sqrt(width))})
    h = rd(rng.standard_normal((n, width)))
    want = O.moe_ff(h, p, mlp)
    t = lambda a, dt=dtype: torch.from_numpy(np.ascontiguousarray(a)).to(device=device, dtype=dt).contiguous()
    rows = [p["router"]] + ([p["shared.sg"]] if shared else [])
    got = moe.grouped_choice_ffn(
        t(h), t(np.concatenate(rows, 0), torch.float32), t(p["correction"], torch.float32),
        t(np.stack([p[f"e{j}.up"] for j in range(e)])), t(np.stack([p[f"e{j}.down"] for j in range(e)])), top, count,
        keep, 1.7, t(p["shared.up"]) if shared else None, t(p["shared.down"]) if shared else None)
    err = np.abs(got.float().cpu().numpy() - want).max(-1) / np.abs(want).max()
    if dtype == torch.float32:
        assert err.max() < 3e-5
    else:
        assert np.median(err) < 2e-2 and (err > 5e-2).mean() <= 0.03


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("width,dim", [(96, 8), (72, 1), (256, 24)])
def test_parallel_add_and_token_input(target, width, dim):
    """x += a + b on the float32 stream, then the per-layer token input (side table columns, gelu gate,
    projection, RMS norm with a plain weight) and the next layer's norm out of the same kernel."""
    device, dtype = _dev(target)
    rng = np.random.default_rng(width)
    n, vocab, layers, li = 19, 50, 3, 1
    rd = lambda a: torch.from_numpy(a.astype(np.float32)).to(dtype)
    x = torch.from_numpy(rng.standard_normal((n, width)).astype(np.float32))
    a, b = rd(rng.standard_normal((n, width))), rd(rng.standard_normal((n, width)))
    table = rd(rng.standard_normal((vocab, layers * dim)))
    gate, proj = rd(rng.standard_normal((dim, width)) / np.sqrt(width)), rd(rng.standard_normal((width, dim)))
    wn, wnext = rd(1 + 0.2 * rng.standard_normal(width)), rd(1 + 0.2 * rng.standard_normal(width))
    ids = rng.integers(0, vocab, n).astype(np.int32)
    xs, xr = lat.par_add(x.clone().to(device), a.to(device), b.to(device), rounded=True)
    want = x.double().numpy() + (a.double().numpy() + b.double().numpy())
    np.testing.assert_allclose(xs.cpu().numpy(), want, atol=2e-6)
    np.testing.assert_allclose(xr.float().cpu().numpy(), want, atol=_atol(dtype, 2e-6, 4e-2))
    xs2, none = lat.par_add(x.clone().to(device), a.to(device))
    assert none is None
    np.testing.assert_allclose(xs2.cpu().numpy(), x.double().numpy() + a.double().numpy(), atol=2e-6)
    from distributed_llms_amd import ops
    z = lat.side_gate(ops.linear(xr, gate.to(device)), table.to(device), torch.from_numpy(ids).to(device), li * dim)
    y = ops.linear(z, proj.to(device))
    xs, hn = sm.post_norm_add(xs, y, wn.to(device), 1e-6, 1.0, w_next=wnext.to(device), one_plus=False)
    e = table.double().numpy()[ids][:, li * dim:(li + 1) * dim]
    pw = {"gate": gate.double().numpy(), "proj": proj.double().numpy(), "norm": wn.double().numpy()}
    want2 = O.token_side(want, e, pw, 1e-6)
    # one column: the norm's input is a multiple of one vector, and where the gate is near zero its
    # size is near sqrt(eps), so float32 rounding of the gate's input shows (an ill-conditioned case)
    f32 = 2e-4 if dim == 1 else 3e-5
    np.testing.assert_allclose(xs.cpu().numpy(), want2, rtol=2e-5, atol=_atol(dtype, f32, 6e-2))
    np.testing.assert_allclose(hn.float().cpu().numpy(), O.rms(want2, wnext.double().numpy(), 1e-6), rtol=2e-5,
                               atol=_atol(dtype, f32, 6e-2))
    cat = lat.stream_cat(xs, xs2, dtype)
    np.testing.assert_allclose(cat.float().cpu().numpy(), np.concatenate([xs.cpu().numpy(), xs2.cpu().numpy()], -1),
                               atol=_atol(dtype, 0, 4e-2))
    np.testing.assert_array_equal(lat.stream_set(cat).cpu().numpy(), cat.float().cpu().numpy())


# ------------------------------------------------------------------------------ the engine
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_prompts_and_layers(target, name, tmp_path):
    cfg = CONFIGS[name]()
    sd = _round(O.make_weights(cfg, seed=3), target[1])
    eng = make_engine(cfg, sd, target, tmp_path)
    prompts = prompts_for(cfg, [1, 2, 45, 130])
    eng.stage.taps = []
    got = replay(eng, [[(n, len(p))] for n, p in prompts.items()], prompts)
    taps = eng.stage.taps
    eng.stage.taps = None
    runs = len(O.layer_runs(cfg))
    for i, (n, p) in enumerate(prompts.items()):
        layers = []
        want = oracle(cfg, sd, p, layers)
        assert_close(got[n], want, target, n, 4.0 if name == "b" else 1.0)
        if target[1] == torch.float32:            # the residual stream after every layer run
            mine = torch.stack(taps[i * runs:(i + 1) * runs]).cpu().numpy()
            np.testing.assert_allclose(mine, np.stack(layers), rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["a", "b"])
def test_decode_and_portions_match_the_whole(target, name, tmp_path):
    """Token-by-token decoding after a prompt (90 steps, over several block borders), portions of
    changing sizes down to two tokens and one, cut inside blocks, and decoding from the very first token."""
    cfg = CONFIGS[name]()
    sd = _round(O.make_weights(cfg, seed=4), target[1])
    eng = make_engine(cfg, sd, target, tmp_path)
    p = prompts_for(cfg, [150], seed=7)
    want = oracle(cfg, sd, p["r0"])
    got = replay(eng, [[("r0", 60)]] + [[("r0", 1)]] * 90, p)
    slack = 4.0 if name == "b" else 1.0
    assert_close(got["r0"], want, target, "decode", slack)
    sizes = [2, 3, 1, 31, 2, 33, 5, 64, 2, 7]
    assert sum(sizes) == 150
    got = replay(eng, [[("r0", s)] for s in sizes], p)
    assert_close(got["r0"], want, target, "portions", slack)
    got = replay(eng, [[("r0", 1)]] * 40, {"r0": p["r0"][:40]})
    assert_close(got["r0"], (want[0][:40], want[1][:40]), target, "from the first token", slack)


@pytest.mark.parametrize("target", TARGETS)
def test_mixed_batches_and_reused_blocks(target, tmp_path):
    """Up to four unequal requests per step, portions beside single tokens; finished requests give
    their blocks to new ones (a pool sized for the live tokens only).  Every request matches its own
    whole-sequence oracle, i.e. the batch and the pool do not show."""
    cfg = cfg_a()
    sd = _round(O.make_weights(cfg, seed=5), target[1])
    eng = make_engine(cfg, sd, target, tmp_path, max_tokens=288, max_requests=4)
    lens = [70, 9, 33, 64, 20, 50, 3]
    prompts = prompts_for(cfg, lens, seed=9)
    names = list(prompts)
    at = {n: 0 for n in names}
    waiting, live, schedule = list(names), [], []
    rng = np.random.default_rng(0)
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        step = []
        for n in list(live):
            left = len(prompts[n]) - at[n]
            c = min(left, int(rng.choice([1, 1, 2, 3, 17, 32])))
            if rng.random() < 0.15 and len(live) > 1:
                continue                                # left out of this step, goes on later
            step.append((n, c))
            at[n] += c
            if at[n] == len(prompts[n]):
                live.remove(n)
        if step:
            schedule.append(step)
    got = replay(eng, schedule, prompts)
    assert eng.bm.num_free() == eng.bm.num_blocks - 1            # all given back (block 0 is the scratch block)
    for n in names:
        assert_close(got[n], oracle(cfg, sd, prompts[n]), target, n)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name,graphs", [("a", False), ("c", True)])
def test_greedy_generation_through_the_scheduler(target, name, graphs, tmp_path):
    """LLMEngine.generate (scheduler, continuous batching, sampler; for the model whose experts the
    grouped kernels take, decode steps replayed from HIP graphs) on three prompts at once: every
    generated token is the argmax of the oracle's logits for the sequence so far (where the oracle's
    top two are not within rounding of each other)."""
    cfg = CONFIGS[name]()
    sd = _round(O.make_weights(cfg, seed=6), target[1])
    eng = make_engine(cfg, sd, target, tmp_path, graphs=graphs)
    prompts = list(prompts_for(cfg, [5, 40, 17], seed=11).values())
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=24, ignore_eos=True))
    margin = 1e-3 if target[1] == torch.float32 else 0.3
    checked = 0
    for p, o in zip(prompts, outs):
        assert len(o) == 24
        logits = O.forward(cfg, sd, np.array(p + o))
        for i, tok in enumerate(o):
            row = logits[len(p) + i - 1]
            top = np.sort(row)[-2:]
            if top[1] - top[0] > margin:
                checked += 1
                assert tok == int(row.argmax()), (i, tok, int(row.argmax()))
    assert checked > (36 if target[1] == torch.float32 else 12)


def test_config_round_trip_and_registry(tmp_path):
    from distributed_llms_amd.config import get_model_config
    from distributed_llms_amd.models.gikovik import GikovikStage, layer_runs, model_shapes
    cfg = cfg_a()
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    m = get_model_config(str(tmp_path))
    assert m.arch == "gikovik" and m.num_layers == 4 and m.hidden_size == 96
    assert m.needs_seq_index and not m.needs_state_slots
    back = ModelConfig.from_hf_config(m.to_hf_config())
    assert back.layers == m.layers and back.loop == m.loop and back.token_side_dim == 8
    assert [i for i, _ in layer_runs(m)] == [0, 1, 2, 1, 2, 3] and [e for _, e in layer_runs(m)] == [0, 1, 0, 1, 0, 0]
    st = make_stage(m)
    assert isinstance(st, GikovikStage) and st.num_layers == 6          # one cache per layer run
    assert {k: tuple(v.shape) for k, v in O.make_weights(cfg).items()} == model_shapes(m)
    plain = ModelConfig.from_hf_config(cfg_c())
    assert plain.loop is None and plain.token_side_dim == 0 and len(layer_runs(plain)) == 2
    for bad in ({"type": "attention"}, {"mlp": {"kind": "glu", "ff": 8}}):
        c = cfg_a()
        c["layers"][0].update(bad)
        with pytest.raises(ValueError):
            ModelConfig.from_hf_config(c)
    c = cfg_a()
    c["loop"]["stop"] = 9
    with pytest.raises(ValueError):
        ModelConfig.from_hf_config(c)
    assert get_model_config("tiny-gikovik").arch == "gikovik"
    make_stage(get_model_config("tiny-gikovik")).init_synthetic(0)


@pytest.mark.parametrize("target", [t for t in TARGETS if "gpu" in t.id])
def test_decode_graphs_replay_like_eager_steps(target, tmp_path):
    """Decode steps replayed from captured HIP graphs (several replays, eager prompt steps and
    synchronisations between them) give the logits of eager decode steps."""
    if target[1] != torch.bfloat16:
        pytest.skip("the float32 expert path reads row counts on the host: it decodes eagerly")
    cfg = cfg_c()
    sd = _round(O.make_weights(cfg, seed=8), target[1])
    p = prompts_for(cfg, [40, 23], seed=3)
    sched = [[("r0", 30), ("r1", 13)]] + [[("r0", 1), ("r1", 1)]] * 10
    eager = replay(make_engine(cfg, sd, target, tmp_path, graphs=False), sched, p)
    eng = make_engine(cfg, sd, target, tmp_path, graphs=True)
    assert eng.runner.graphs is not None
    graphed = replay(eng, sched, p)
    for n in p:
        np.testing.assert_allclose(graphed[n], eager[n], rtol=1e-3, atol=1e-3)
