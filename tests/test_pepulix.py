"""The Pepulix decoder in the engine against the plain implementation (`plain_pepulix.py`).

Each mechanism alone (the kernel of the residual streams, per-head norms with rotation and value mixing, the
matrix memory's scan with its state rows, the heads' norm with a sigmoid gate, the softmax router, gated experts
beside experts that hand their input on, one-layer models of every mixer and feed-forward), keys placed so that
one far score stands out, a memory that never forgets through one reused slot, then whole models under every
way of cutting and batching over poisoned pages and stale slots, the stream after every layer, replays against
unrecorded steps, and greedy generation through the engine, the command line and the replay program.  The tests
make their own small configurations and weights; sizes differ from layer to layer, also where a model could make
them equal, and some are 1.

`double` cases run everything above the kernels on the CPU stand-in; `hip` cases run the HIP kernels
(`-m gpu`) in float32 and bfloat16.
"""

from __future__ import annotations

import copy
import json
import math
from pathlib import Path
from types import SimpleNamespace

import pytest
import torch

import mini_llm_runtime_amd.models  # noqa: F401
import plain_pepulix as plain
import schedules
from helpers import StepEntry, make_runner, random_tokens
from kernel_doubles import TorchOps
from mini_llm_runtime_amd.config import ConfigError
from mini_llm_runtime_amd.config.pepulix import PepulixConfig
from mini_llm_runtime_amd.engine import ContinuousBatchEngine
from mini_llm_runtime_amd.models import build_model, config_from_dict
from mini_llm_runtime_amd.weights import save_state_dict

ROOT = Path(__file__).resolve().parents[1]


# ---- configurations -----------------------------------------------------------------------------------

def _rot(base, dims, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling is not None:
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return out


def _attn(heads, kv_heads, dim, vdim, scale, rot=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        m["rot"] = rot
    if v_mix:
        m["v_mix"] = True
    return "attention", m


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot):
    return "latent_attention", {
        "heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
        "rot": rot,
    }


def _memory(heads, dim, vdim, cap):
    return "mlstm", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, experts, identity, top):
    router = {"experts": experts, "top": top}
    if identity:
        router["identity"] = identity
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def _model(vocab, width, eps, layers, streams=None, softcap=None):
    cfg = {
        "architecture": "Pepulix", "vocab": vocab, "width": width, "norm": {"eps": eps},
        "layers": [{"type": kind, "mixer": mixer, "mlp": mlp} for (kind, mixer), mlp in layers],
    }
    if streams is not None:
        cfg["streams"] = streams
    if softcap is not None:
        cfg["logit_softcap"] = softcap
    return cfg


YARN = (4.0, 64, 16.0, 1.0)
CONFIGS = {
    # every mixer and feed-forward, three streams, values mixed between two attention layers of other head counts
    "A": _model(97, 64, 1e-5, [
        (_latent(2, 16, 8, 24, 32, 24, 0.3, _rot(10000.0, 8, YARN)), _dense(96)),
        (_memory(2, 16, 32, 10.0), _moe(40, 6, 2, 2)),
        (_attn(4, 2, 32, 16, 0.2, _rot(5000.0, 16), v_mix=True), _moe(24, 4, 0, 3)),
        (_memory(4, 8, 8, 15.0), None),
        (_attn(2, 2, 16, 16, 0.25, _rot(300.0, 16), v_mix=True), _dense(72)),
        (_attn(6, 2, 16, 16, 0.25, None, v_mix=True), None),
    ], streams=3, softcap=12.0),
    # one stream kept as hyper-connections, one head everywhere, every expert chosen, widths no kernel likes
    "B": _model(61, 36, 1e-6, [
        (_attn(1, 1, 20, 20, 0.22), _moe(10, 2, 1, 3)),
        (_latent(1, 12, 6, 10, 20, 9, 0.25, _rot(100.0, 4)), _dense(27)),
        (_memory(1, 20, 12, 5.0), _dense(16)),
    ], streams=1, softcap=30.0),
    # no `streams` at all (plain additions), no cap, only experts that hand their input on may be chosen
    "C": _model(128, 48, 1e-5, [
        (_memory(3, 16, 16, 15.0), _moe(32, 3, 5, 2)),
        (_latent(3, 16, 16, 16, 48, 32, 0.2, _rot(500000.0, 16, (8.0, 32, 32.0, 2.0))), None),
        (_attn(3, 1, 48, 64, 0.15, _rot(20000.0, 24)), _dense(64)),
    ]),
    # long requests: decode partitions, many key tiles, a state walked over hundreds of tokens
    "D": _model(80, 64, 1e-5, [
        (_attn(4, 2, 32, 32, 0.3, _rot(10000.0, 32), v_mix=True), _dense(64)),
        (_latent(4, 16, 16, 16, 48, 16, 0.3, _rot(10000.0, 16, YARN)), None),
        (_memory(2, 32, 32, 15.0), None),
        (_attn(4, 2, 32, 32, 0.3, _rot(10000.0, 32), v_mix=True), None),
    ], streams=2, softcap=15.0),
}
BLOCK = {"A": 16, "B": 8, "C": 4, "D": 16}
LENGTHS = {"A": (1, 9, 50, 83, 37, 64), "B": (2, 19, 35, 66, 45), "C": (5, 17, 140, 70), "D": (660, 341)}


def make_weights(cfg: dict, seed: int) -> dict[str, torch.Tensor]:
    """bfloat16 tensors by the design's checkpoint names, larger than an initialisation would be."""
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]
    streams = cfg.get("streams")

    def normal(*shape, std, mean=0.0):
        return (torch.randn(shape, generator=g) * std + mean).to(torch.bfloat16)

    def matrix(rows, cols, gain=1.0):
        return normal(rows, cols, std=gain / math.sqrt(cols))

    w = {"embed": normal(cfg["vocab"], width, std=1.0), "final.norm": normal(width, std=0.2, mean=1.0)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"] = normal(width, std=0.2, mean=1.0)
        out = m["heads"] * m["vdim"]
        if layer["type"] == "attention":
            kv = m.get("kv_heads", m["heads"])
            w[p + "mix.q"] = matrix(m["heads"] * m["dim"], width)
            w[p + "mix.k"] = matrix(kv * m["dim"], width)
            w[p + "mix.v"] = matrix(kv * m["vdim"], width)
            for n, rows in (("q", m["heads"] * m["dim"]), ("k", kv * m["dim"]), ("v", kv * m["vdim"])):
                w[p + f"mix.{n}.b"] = normal(rows, std=0.3)
            w[p + "mix.pb"] = normal(m["heads"], std=1.0, mean=-1.5)
            w[p + "mix.g"] = matrix(m["heads"], width, 1.5)
            if m.get("v_mix"):
                w[p + "mix.vmix"] = normal(std=0.1, mean=0.4)
        elif layer["type"] == "latent_attention":
            w[p + "mix.dq"] = matrix(m["q_rank"], width)
            w[p + "mix.dq.norm"] = normal(m["q_rank"], std=0.2, mean=1.0)
            w[p + "mix.uq"] = matrix(m["heads"] * (m["dim"] + m["rot_dim"]), m["q_rank"], 2.0)
            w[p + "mix.dkv"] = matrix(m["kv_rank"] + m["rot_dim"], width, 2.0)
            w[p + "mix.dkv.norm"] = normal(m["kv_rank"], std=0.2, mean=1.0)
            w[p + "mix.uk"] = matrix(m["heads"] * m["dim"], m["kv_rank"], 2.0)
            w[p + "mix.uv"] = matrix(out, m["kv_rank"])
        else:
            w[p + "mix.q"] = matrix(m["heads"] * m["dim"], width)
            w[p + "mix.k"] = matrix(m["heads"] * m["dim"], width)
            w[p + "mix.v"] = matrix(out, width)
            w[p + "mix.g"] = matrix(out, width, 1.5)
            w[p + "mix.norm"] = normal(out, std=0.2, mean=1.0)
            w[p + "mix.i"] = matrix(m["heads"], width, 2.0)
            w[p + "mix.i.b"] = normal(m["heads"], std=1.0)
            w[p + "mix.f"] = matrix(m["heads"], width, 2.0)
            w[p + "mix.f.b"] = normal(m["heads"], std=1.0, mean=2.0)
        w[p + "mix.o"] = matrix(width, out)
        f = layer["mlp"]
        sublayers = ["hc1"]
        if f is not None:
            sublayers.append("hc2")
            w[p + "norm2"] = normal(width, std=0.2, mean=1.0)
            if f["kind"] == "dense":
                w[p + "mlp.gate"] = matrix(f["ff"], width, 1.5)
                w[p + "mlp.up"] = matrix(f["ff"], width, 1.5)
                w[p + "mlp.down"] = matrix(width, f["ff"])
                w[p + "mlp.gate.b"] = normal(f["ff"], std=0.3)
                w[p + "mlp.up.b"] = normal(f["ff"], std=0.3)
                w[p + "mlp.down.b"] = normal(width, std=0.3)
            else:
                r = f["router"]
                routed = r["experts"] + r.get("identity", 0)
                w[p + "mlp.router"] = matrix(routed, width, 2.5)
                w[p + "mlp.correction"] = normal(routed, std=0.1)
                for e in range(r["experts"]):
                    w[p + f"mlp.e{e}.gate"] = matrix(f["expert"]["ff"], width, 1.5)
                    w[p + f"mlp.e{e}.up"] = matrix(f["expert"]["ff"], width, 1.5)
                    w[p + f"mlp.e{e}.down"] = matrix(width, f["expert"]["ff"])
        if streams is not None:
            for hc in sublayers:
                w[p + hc + ".in"] = normal(streams, std=0.3, mean=0.7)
                w[p + hc + ".out"] = normal(streams, std=0.3, mean=0.8)
                w[p + hc + ".mix"] = (torch.eye(streams) + 0.25 * torch.randn(streams, streams, generator=g)).to(torch.bfloat16)
    return w


def write_model(tmp_path, name: str, cfg: dict, weights: dict) -> Path:
    folder = Path(tmp_path) / name
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_state_dict(folder / "model.safetensors", weights)
    return folder


def make_dir(tmp_path, which: str, seed: int = 3):
    cfg = CONFIGS[which]
    weights = make_weights(cfg, seed)
    return write_model(tmp_path, f"pepulix{which}", cfg, weights), cfg, weights


def _f64(weights):
    return {k: v.to(torch.float64) for k, v in weights.items()}


def _ops(backend: str, dtype: torch.dtype):
    if backend == "double":
        return TorchOps(dtype, "cpu")
    from mini_llm_runtime_amd.kernels.ops import HipOps

    return HipOps(dtype, "cuda")


CASES = [
    pytest.param("double", torch.float32, id="double-f32"),
    pytest.param("hip", torch.float32, id="hip-f32", marks=pytest.mark.gpu),
    pytest.param("hip", torch.bfloat16, id="hip-bf16", marks=pytest.mark.gpu),
]
GPU_CASES = [
    pytest.param(torch.float32, id="f32", marks=pytest.mark.gpu),
    pytest.param(torch.bfloat16, id="bf16", marks=pytest.mark.gpu),
]


CLOSE_CALL = 2.5e-2  # of a router's choice scores (probabilities plus a correction): what the bfloat16 stream's error of a percent or two moves them by


def _compare(got, requests, weights, cfg, dtype, f32_bound=1e-4, row_bound=6e-2, together=3e-2):
    """float32: every value within 1e-4 of the logits' size.  bfloat16: all rows together within 3 % (relative
    L2, the mean over the vocabulary taken off); every row within 6 %, but for a few (one in twenty, and as many
    as rounding alone puts beyond 6 %) that may be off by up to 4 times what rounding alone does to the worst row
    of their request (the plain implementation with the inputs of its products rounded to bfloat16): where a
    router's two candidates are nearly tied, or a memory's denominator is near its floor, rounding moves a row
    by percents in the plain implementation as in the engine.  A wrong key, page, slot, state or expert changes
    most rows, by half and more.  Rows at which a router's choice is a close call in the plain implementation
    (the last chosen expert leads the first one left out by less than `CLOSE_CALL`) are left out in bfloat16:
    there the engine's own roundings may send the token to the other expert while the rounded plain implementation
    happens not to, and the two experts' weights can differ by a quarter of the row."""
    assert got, "no logits came back"
    w64 = _f64(weights)
    num = den = 0.0
    loose = rows = loose_alone = 0
    for rid, toks in requests.items():
        notes: dict = {}
        ref, _ = plain.forward(cfg, w64, toks, notes=notes)
        close = torch.zeros(len(toks), dtype=torch.bool)
        for margin in notes.get("margins", []):
            close |= margin.abs() < CLOSE_CALL
        ref = ref - ref.mean(-1, keepdim=True)
        size = float(ref.pow(2).mean().sqrt())
        if dtype != torch.float32:
            coarse, _ = plain.forward(cfg, w64, toks, round_to=torch.bfloat16)
            coarse = coarse - coarse.mean(-1, keepdim=True)
            alone = (coarse - ref).pow(2).sum(-1).sqrt() / ref.pow(2).sum(-1).sqrt()
            loose_alone += int((alone >= row_bound).sum())
        for pos in range(len(toks)):
            row = got[(rid, pos)].double()
            assert torch.isfinite(row).all(), f"{rid}:{pos} is not finite"
            diff = row - row.mean() - ref[pos]
            if dtype == torch.float32:
                assert float(diff.abs().max()) < f32_bound * size, f"{rid}:{pos}: off by {float(diff.abs().max()):.3e} of {size:.3e}"
                continue
            rows += 1
            rel = float(diff.pow(2).sum().sqrt() / ref[pos].pow(2).sum().sqrt())
            if rel >= row_bound and bool(close[pos]):
                continue
            if rel >= row_bound:
                loose += 1
                assert rel < 4.0 * max(float(alone.max()), row_bound / 2), f"{rid}:{pos}: relative error {rel:.3e}, rounding alone up to {float(alone.max()):.3e}"
                continue
            num += float(diff.pow(2).sum())
            den += float(ref[pos].pow(2).sum())
    if dtype != torch.float32:
        assert loose <= 0.05 * rows + 1 + 1.5 * loose_alone, f"{loose} of {rows} rows are off by more than {row_bound}, {loose_alone} by rounding alone"
        assert (num / den) ** 0.5 < together, f"relative error of all rows {(num / den) ** 0.5:.3e}"


def _requests(which: str) -> dict[str, list[int]]:
    vocab = CONFIGS[which]["vocab"]
    return {f"r{i}": random_tokens(n, vocab, 50 + i) for i, n in enumerate(LENGTHS[which])}


# ---- configuration and model --------------------------------------------------------------------------

def test_config_reads_every_layer_by_itself():
    c = config_from_dict(CONFIGS["A"])
    assert isinstance(c, PepulixConfig)
    assert [l.mixer.kind for l in c.layers] == ["latent_attention", "mlstm", "attention", "mlstm", "attention", "attention"]
    assert c.streams == 3 and c.logit_softcap == 12.0
    assert c.layers[0].mixer.q_rank == 24 and c.layers[0].mixer.rot.scaling.factor == 4.0
    assert c.layers[1].mlp.kind == "moe" and (c.layers[1].mlp.experts, c.layers[1].mlp.identity, c.layers[1].mlp.top) == (6, 2, 2)
    assert c.layers[2].mixer.v_mix and c.layers[2].mixer.kv_heads == 2 and c.layers[3].mlp is None
    assert c.layers[5].mixer.rot is None
    assert PepulixConfig.from_dict(c.to_dict()) == c
    plain_config = config_from_dict(CONFIGS["C"])
    assert plain_config.streams is None and plain_config.logit_softcap is None


@pytest.mark.parametrize(
    "change",
    [
        lambda c: c["layers"][0]["mixer"].pop("q_rank"),
        lambda c: c["layers"][0].update(type="convolution"),
        lambda c: c["layers"][2]["mixer"].update(kv_heads=3),  # four heads on three
        lambda c: c["layers"][2]["mixer"]["rot"].update(dims=40),  # more than a head has
        lambda c: c["layers"][4]["mixer"].update(vdim=8),  # mixed values of two widths
        lambda c: c["layers"][1]["mlp"]["router"].update(top=9),  # more than there are
        lambda c: c["layers"][1]["mlp"].update(kind="sparse"),
        lambda c: c.update(streams=0),
        lambda c: c.update(logit_softcap=-1.0),
        lambda c: c["layers"][1]["mixer"].update(gate_cap=0),
    ],
)
def test_config_refuses_what_does_not_fit(change):
    cfg = copy.deepcopy(CONFIGS["A"])
    change(cfg)
    with pytest.raises(ConfigError):
        config_from_dict(cfg)


def test_model_is_built_from_the_framework_parts():
    from mini_llm_runtime_amd.parts.block import HyperConnectionBlock, PreNormBlock
    from mini_llm_runtime_amd.parts.feed_forward import RoutedExperts, SwiGLU
    from mini_llm_runtime_amd.parts.latent_attention import LatentAttention
    from mini_llm_runtime_amd.parts.matrix_memory import MatrixMemory
    from mini_llm_runtime_amd.parts.sigmoid_attention import SigmoidAttention

    model = build_model(config_from_dict(CONFIGS["A"]))
    assert all(isinstance(layer, HyperConnectionBlock) and layer.streams == 3 for layer in model.layers)
    assert [type(layer.mixer) for layer in model.layers] == [
        LatentAttention, MatrixMemory, SigmoidAttention, MatrixMemory, SigmoidAttention, SigmoidAttention
    ]
    assert [layer.mixer.value_source for layer in model.layers if isinstance(layer.mixer, SigmoidAttention)] == ["first", "mixed", "mixed"]
    assert isinstance(model.layers[0].feed_forward, SwiGLU) and model.layers[0].feed_forward.bias
    experts = model.layers[1].feed_forward
    assert isinstance(experts, RoutedExperts) and (experts.scores, experts.normalise, experts.identity) == ("softmax", True, 2)
    assert model.layers[3].feed_forward is None and model.spec.tie_word_embeddings and model.spec.residual_streams == 3
    assert model.replayable and model.splittable
    # the memory keeps its state in the manager's slots, the attentions their keys in pages
    kinds = [type(s).__name__ for s in model.site_cache_specs()]
    assert kinds == ["PagedKVSpec", "SlotStateSpec", "PagedKVSpec", "SlotStateSpec", "PagedKVSpec", "PagedKVSpec"]
    assert all(isinstance(layer, PreNormBlock) for layer in build_model(config_from_dict(CONFIGS["C"])).layers)


# ---- mechanisms alone, on the GPU ------------------------------------------------------------------------

def _tolerance(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("streams,tokens,width,slices", [(1, 1, 64, 0), (3, 7, 100, 3), (4, 300, 208, 0), (2, 5, 2048, 2), (16, 9, 72, 1), (2, 3, 70, 0), (2, 2, 4104, 0), (4, 3, 4096, 1)])
def test_streams_step(dtype, streams, tokens, width, slices):
    """Update, weighted sum and norm in one kernel, against the formulas; on chosen rows the streams stay."""
    ops = _ops("hip", dtype)
    g = torch.Generator().manual_seed(streams * 100 + tokens)
    x = torch.randn(streams, tokens, width, generator=g)
    y = torch.randn(max(slices, 1), tokens, width, generator=g)
    mix = torch.eye(streams) + 0.3 * torch.randn(streams, streams, generator=g)
    write, read = torch.randn(streams, generator=g), torch.randn(streams, generator=g)
    weight = 1 + 0.2 * torch.randn(width, generator=g)
    y_sum = y.sum(0) if slices else y[0].to(dtype).float()
    new = torch.einsum("st,snw->tnw", mix.double(), x.double()) + write.double()[:, None, None] * y_sum.double()[None]
    u = torch.einsum("s,snw->nw", read.double(), new)
    h = u / torch.sqrt((u * u).mean(-1, keepdim=True) + 1e-5) * weight.double()
    dev = lambda t: t.cuda().contiguous()
    xd = dev(x)
    y_dev = dev(y) if slices else dev(y[0].to(dtype))
    got, total = ops.streams_step(
        xd, update=(y_dev, dev(mix), dev(write)), read_weights=dev(read), norm_weight=dev(weight), eps=1e-5, want_sum=True
    )
    torch.testing.assert_close(xd.cpu().double(), new, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(total.cpu().double(), u, rtol=1e-5, atol=2e-5)
    torch.testing.assert_close(got.cpu().double(), h, **_tolerance(dtype))
    # chosen rows, the plain sum, no norm: the streams are left alone
    rows = torch.tensor([tokens - 1, 0], dtype=torch.int32).cuda()
    xd = dev(x)
    none, total = ops.streams_step(xd, update=(y_dev, dev(mix), dev(write)), rows=rows, want_sum=True)
    assert none is None and torch.equal(xd.cpu(), x)
    torch.testing.assert_close(total.cpu().double(), new.sum(0)[[tokens - 1, 0]], rtol=1e-5, atol=2e-5)
    assert torch.equal(ops.streams_fill(dev(x[0]), streams).cpu(), x[0][None].repeat(streams, 1, 1))


def _step_context(lengths, starts, ops):
    cu = [0]
    for n in lengths:
        cu.append(cu[-1] + n)
    dev = ops.device
    return SimpleNamespace(
        num_entries=len(lengths), cu_q=torch.tensor(cu, dtype=torch.int32, device=dev),
        q_starts=torch.tensor(starts, dtype=torch.int32, device=dev),
    )


@pytest.mark.gpu
@pytest.mark.parametrize("in_runs", [False, True], ids=["whole", "in-runs"])
@pytest.mark.parametrize("heads,dim,vdim", [(2, 16, 32), (3, 20, 12), (4, 64, 48), (1, 128, 70), (2, 200, 20), (1, 1, 1)])
def test_memory_scan_and_its_state_rows(heads, dim, vdim, in_runs):
    """Entries of 1, 5 and 150 tokens (three runs, the last not full), one that starts its request on a row full of NaN, two that go on from a
    carried state; rows that no entry writes stay as they were.  Against the stand-in's loop over tokens, which
    the CPU tests hold against the plain implementation."""
    hip, double = _ops("hip", torch.float32), TorchOps(torch.float32, "cpu")
    g = torch.Generator().manual_seed(heads * 1000 + dim)
    lengths, starts = [1, 5, 150], [3, 0, 9]
    tokens = sum(lengths)
    qk, v = heads * dim, heads * vdim
    width = 2 * qk + 2 * v + 2 * heads + 3  # something behind the gates too
    offsets = (v, v + qk, 0, 2 * qk + 2 * v + 1, 2 * qk + 2 * v + 1 + heads)  # values first, a gap before the gates
    projected = torch.randn(tokens, width, generator=g)
    projected[:, offsets[3] :] *= 3.0
    state = torch.randn(8, heads, dim * vdim + dim + 1, generator=g) * 0.5
    state[5] = float("nan")
    read = torch.tensor([2, 5, 6], dtype=torch.int32)
    write = torch.tensor([3, 4, 7], dtype=torch.int32)
    want_state = state.clone()
    want = double.matrix_memory_scan(
        projected, want_state, read, write, _step_context(lengths, starts, double), heads=heads, head_dim=dim,
        value_dim=vdim, offsets=offsets, cap=6.0, q_scale=dim**-0.5,
    )
    got_state = state.cuda()
    got = hip.matrix_memory_scan(
        projected.cuda(), got_state, read.cuda(), write.cuda(), _step_context(lengths, starts, hip), heads=heads,
        head_dim=dim, value_dim=vdim, offsets=offsets, cap=6.0, q_scale=dim**-0.5, in_runs=in_runs,
    )
    torch.testing.assert_close(got.cpu(), want, rtol=2e-4, atol=2e-4)
    torch.testing.assert_close(got_state.cpu(), want_state, rtol=2e-4, atol=2e-4, equal_nan=True)
    for row in (0, 1, 2, 5, 6):
        assert torch.equal(got_state[row].cpu().nan_to_num(7.0), state[row].nan_to_num(7.0))


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("heads,kv,dim,vdim,rdims,block", [(4, 2, 32, 16, 16, 8), (1, 1, 20, 20, 0, 4), (6, 3, 16, 40, 16, 16), (2, 2, 128, 32, 64, 16)])
def test_head_norms_rotation_and_value_mixing(dtype, heads, kv, dim, vdim, rdims, block):
    hip, double = _ops("hip", dtype), TorchOps(dtype, "cpu")
    g = torch.Generator().manual_seed(heads + dim)
    tokens = 37
    pages = -(-tokens // block) + 1
    D = -(-max(dim, vdim) // 16) * 16
    width = (heads + kv) * dim + kv * vdim + heads
    projected = torch.randn(tokens, width, generator=g) * 2.0
    rotation = None
    if rdims:
        angle = torch.rand(tokens, rdims // 2, generator=g) * 6.0
        rotation = (torch.cos(angle), torch.sin(angle), rdims)
    slots = torch.randperm(pages * block, generator=g)[:tokens].to(torch.int32)
    slots[3] = -1
    first = torch.randn(tokens, kv * vdim, generator=g)
    lam = torch.tensor([0.35])
    results = []
    for ops in (double, hip):
        to = (lambda t: t.cuda()) if ops is hip else (lambda t: t)
        keys = to(torch.zeros(pages, kv, block, D, dtype=dtype))
        values = to(torch.zeros(pages, kv, D, block, dtype=dtype))
        common = dict(
            heads=heads, kv_heads=kv, head_dim=dim, value_dim=vdim, kernel_dim=D, eps=1e-5,
            rotation=None if rotation is None else (to(rotation[0]), to(rotation[1]), rdims), slot_mapping=to(slots),
            key_pages=keys, value_pages=values, block_size=block,
        )
        q, gate, kept = ops.head_norm_rope_write(to(projected), gated=True, keep_values=True, **common)
        plain_values = values.clone()
        q2, _, none = ops.head_norm_rope_write(to(projected), gated=True, first_values=to(first), mix_weight=to(lam), **common)
        assert none is None
        results.append([t.float().cpu() for t in (q, gate, kept, keys, plain_values, q2, values)])
    for a, b in zip(*results):
        torch.testing.assert_close(b, a, **_tolerance(dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("tokens,experts,top", [(1, 4, 1), (33, 16, 3), (70, 7, 7), (5, 130, 6)])
def test_softmax_router_with_normalised_weights(tokens, experts, top):
    hip, double = _ops("hip", torch.float32), TorchOps(torch.float32, "cpu")
    g = torch.Generator().manual_seed(tokens + experts)
    logits = torch.randn(tokens, experts, generator=g) * 3.0
    correction = torch.randn(experts, generator=g) * 0.2
    want_ids, want = double.route_experts(logits, correction, top=top, groups=1, keep_groups=1, scale=1.0, scores="softmax", normalise=True)
    ids, weights = hip.route_experts(logits.cuda(), correction.cuda(), top=top, groups=1, keep_groups=1, scale=1.0, scores="softmax", normalise=True)
    assert torch.equal(ids.cpu(), want_ids)
    torch.testing.assert_close(weights.cpu(), want, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(weights.sum(-1).cpu(), torch.ones(tokens), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", GPU_CASES)
@pytest.mark.parametrize("tokens,hidden,inner,experts,extra,top", [(1, 64, 24, 4, 2, 2), (70, 40, 10, 3, 1, 3), (300, 64, 32, 2, 5, 2), (9, 36, 7, 5, 0, 1)])
def test_gated_experts_beside_experts_that_hand_on(dtype, tokens, hidden, inner, experts, extra, top):
    hip, double = _ops("hip", dtype), TorchOps(dtype, "cpu")
    g = torch.Generator().manual_seed(tokens + hidden)
    h = torch.randn(tokens, hidden, generator=g).to(dtype)
    up = (torch.randn(experts * 2 * inner, hidden, generator=g) / math.sqrt(hidden)).to(dtype)
    down = (torch.randn(experts * hidden, inner, generator=g) / math.sqrt(inner)).to(dtype)
    ids = torch.stack([torch.randperm(experts + extra, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    weights = torch.rand(tokens, top, generator=g)
    want = double.expert_products(h, up, down, ids, weights, experts=experts, activation="swiglu", pass_through=extra)
    got = hip.expert_products(h.cuda(), up.cuda(), down.cuda(), ids.cuda(), weights.cuda(), experts=experts, activation="swiglu", pass_through=extra)
    torch.testing.assert_close(got.cpu(), want, **_tolerance(dtype))


@pytest.mark.parametrize("dtype", GPU_CASES)
def test_heads_norm_with_a_weight_over_all_heads_and_a_sigmoid_gate(dtype):
    hip, double = _ops("hip", dtype), TorchOps(dtype, "cpu")
    g = torch.Generator().manual_seed(5)
    for heads, vdim in ((3, 20), (1, 48), (4, 64)):
        retained = torch.randn(19, heads * vdim, generator=g)
        projected = torch.randn(19, 7 + heads * vdim, generator=g)
        weight = 1 + 0.3 * torch.randn(heads * vdim, generator=g)
        kw = dict(heads=heads, value_dim=vdim, gate_offset=7, eps=1e-5, gate="sigmoid")
        want = double.retention_gate(retained, projected, norm_weight=weight, **kw)
        got = hip.retention_gate(retained.cuda(), projected.cuda(), norm_weight=weight.cuda(), **kw)
        torch.testing.assert_close(got.float().cpu(), want.float(), **_tolerance(dtype))


# ---- one layer of each kind ----------------------------------------------------------------------------------

ONE_LAYER = {
    "attention": (_attn(4, 2, 16, 24, 0.3, _rot(1000.0, 8)), None),
    "attention-plain": (_attn(2, 2, 8, 8, 0.4), None),
    "latent": (_latent(3, 8, 8, 12, 24, 16, 0.3, _rot(1000.0, 6, YARN)), None),
    "memory": (_memory(2, 12, 20, 8.0), None),
    "dense": (_memory(1, 8, 8, 8.0), _dense(40)),
    "experts": (_memory(1, 8, 8, 8.0), _moe(16, 5, 3, 3)),
}


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("streams", [None, 2])
@pytest.mark.parametrize("kind", list(ONE_LAYER))
def test_one_layer_of_each_kind(tmp_path, kind, streams, backend, dtype):
    cfg = _model(50, 32, 1e-5, [ONE_LAYER[kind]], streams=streams, softcap=8.0)
    weights = make_weights(cfg, 21)
    folder = write_model(tmp_path, "one", cfg, weights)
    requests = {"a": random_tokens(45, 50, 3), "b": random_tokens(1, 50, 4)}
    _, _, cache, runner = make_runner(folder, _ops(backend, dtype), block_size=8, num_blocks=8, max_requests=2)
    cache.poison()
    for family in (schedules.whole, lambda r: schedules.bulk_then_tail(r, tail=9), schedules.portions):
        _compare(schedules.run_schedule(runner, cache, family(requests)), requests, weights, cfg, dtype)


# ---- keys far away and at page borders ------------------------------------------------------------------------

def _needle_model(dim: int, streams):
    """One attention layer, one head, whose query and key are the normed input itself, a bias that shuts every
    key out and a scale that lets in only a key equal to the query: a token's output is the sum of the values of
    the earlier tokens with its own id (itself included), so ONE far key doubles it."""
    cfg = _model(40, dim, 1e-6, [(_attn(1, 1, dim, dim, 1.0), None)], streams=streams)
    weights = make_weights(cfg, 2)
    eye = torch.eye(dim).to(torch.bfloat16)
    weights["l0.mix.q"], weights["l0.mix.k"] = eye.clone(), eye.clone()
    weights["l0.mix.q.b"] = torch.zeros(dim, dtype=torch.bfloat16)
    weights["l0.mix.k.b"] = torch.zeros(dim, dtype=torch.bfloat16)
    weights["l0.norm1"] = torch.ones(dim, dtype=torch.bfloat16)
    weights["l0.mix.pb"] = torch.tensor([-0.6 * dim], dtype=torch.bfloat16)  # equal: +0.4 dim; unrelated: about -0.6 dim
    weights["l0.mix.g"] = torch.zeros(1, dim, dtype=torch.bfloat16)
    return cfg, weights


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("length,marked", [(70, 0), (200, 15), (700, 16), (131, 63), (97, 95)])
def test_one_far_key_that_doubles_the_output(tmp_path, backend, dtype, length, marked):
    if backend == "double" and length > 300:
        pytest.skip("the CPU stand-in is slow at this size")
    cfg, weights = _needle_model(32, 2)
    folder = write_model(tmp_path, "needle", cfg, weights)
    toks = [1 + (i % 30) for i in range(length)]  # ids 1..30 in turn
    toks[marked] = 39
    toks[-1] = 39  # the last token asks for the marked one
    other = list(toks)
    other[marked] = 38
    w64 = _f64(weights)
    with_key, without = plain.forward(cfg, w64, toks)[0][-1], plain.forward(cfg, w64, other)[0][-1]
    assert float((with_key - without).abs().max()) > 0.2 * float(with_key.abs().max()), "the oracle does not see the key"
    _, _, cache, runner = make_runner(folder, _ops(backend, dtype), block_size=16, num_blocks=-(-length // 16), max_requests=1)
    cache.poison()
    cut = max(1, length - 5)
    for steps in (
        schedules.whole({"a": toks}),  # the asking token at the end of a prompt
        schedules.bulk_then_tail({"a": toks}, tail=3),  # decoded alone
        schedules.portions({"a": toks}, sizes=(cut - 1, 2, 3, 2)),  # at the end of a short portion
    ):
        got = schedules.run_schedule(runner, cache, steps)
        row = got[("a", length - 1)].double()
        err = float((row - with_key).abs().max())
        assert err < (1e-4 if dtype == torch.float32 else 5e-2) * float(with_key.abs().max()), err


@pytest.mark.parametrize("backend,dtype", CASES)
def test_a_memory_that_never_forgets_through_one_slot(tmp_path, backend, dtype):
    """A forget gate held open: the first token's key and value stay in the state for good, so a state lost
    between two steps, or a slot cleared too late or not at all, shows at every later position."""
    cfg = _model(64, 32, 1e-6, [(_memory(2, 8, 16, 12.0), None)], streams=2)
    weights = make_weights(cfg, 11)
    weights["l0.mix.f.b"] = torch.full((2,), 40.0, dtype=torch.bfloat16)  # f = logsigmoid(12 tanh(..)) = -6e-6
    weights["l0.mix.i.b"] = torch.full((2,), -1.0, dtype=torch.bfloat16)
    weights["l0.mix.i"] = torch.zeros(2, 32, dtype=torch.bfloat16)
    folder = write_model(tmp_path, "keeper", cfg, weights)
    a = random_tokens(90, 64, 1)
    b = [(a[0] + 1) % 64] + a[1:]  # differs in the first token only
    w64 = _f64(weights)
    ref_a, ref_b = plain.forward(cfg, w64, a)[0], plain.forward(cfg, w64, b)[0]
    assert float((ref_a[20] - ref_b[20]).abs().max()) > 0.03 * float(ref_a[20].abs().max())
    assert float((ref_a[-1] - ref_b[-1]).abs().max()) > 0.005 * float(ref_a[-1].abs().max())
    ops = _ops(backend, dtype)
    _, _, cache, runner = make_runner(folder, ops, block_size=8, num_blocks=1, max_requests=1)
    for family in (schedules.whole, lambda r: schedules.bulk_then_tail(r, tail=40), schedules.portions):
        for name, toks in (("a", a), ("b", b), ("a", a)):  # one slot, used again and again
            got = schedules.run_schedule(runner, cache, family({name: toks}))
            _compare(got, {name: toks}, weights, cfg, dtype)


# ---- whole models under every schedule -------------------------------------------------------------------

FAMILIES = {
    "whole": schedules.whole,
    "bulk_then_tail": lambda r: schedules.bulk_then_tail(r, tail=48),
    "portions": schedules.portions,
    "mixed": schedules.mixed,
    "mixed_two_slots": lambda r: schedules.mixed(r, max_live=2, seed=5, decode_tail=20),
}


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("family", list(FAMILIES))
@pytest.mark.parametrize("which", list(CONFIGS))
def test_schedule_matches_plain(tmp_path, which, family, backend, dtype):
    if backend == "double" and (which == "D" or (which in ("A", "C") and family not in ("mixed", "portions"))):
        pytest.skip("the CPU stand-in is slow at this size")
    folder, cfg, weights = make_dir(tmp_path, which)
    requests = _requests(which)
    steps = FAMILIES[family](requests)
    bs = BLOCK[which]
    _, model, cache, runner = make_runner(
        folder, _ops(backend, dtype), block_size=bs, num_blocks=max(1, schedules.pages_needed(steps, bs)),
        max_requests=schedules.most_live(steps),
    )
    cache.poison()
    for bank in cache.state_banks.values():  # stale states in every slot: a request must start from zeros
        bank.tensor.fill_(float("nan"))
    got = schedules.run_schedule(runner, cache, steps)
    _compare(got, requests, weights, cfg, dtype)
    cache.check_invariants()
    assert all(g.allocator.free_count == g.num_blocks for g in cache.groups), "pages were not given back"


@pytest.mark.parametrize("dtype", GPU_CASES)
def test_long_decoding(tmp_path, dtype):
    """Two hundred tokens decoded one by one behind a prompt (replayed steps, partitions of the keys that grow,
    page after page taken, the memory's state swapped at every commit), two requests side by side."""
    folder, cfg, weights = make_dir(tmp_path, "D")
    requests = {"a": random_tokens(330, cfg["vocab"], 21), "b": random_tokens(263, cfg["vocab"], 22)}
    steps = []
    for pos in range(330):  # a's prompt of 130 and b's of 63 in one step each, then a token of each per step
        entries = []
        for rid, toks in requests.items():
            head = len(toks) - 200
            if pos == head - 1:
                entries.append({"id": rid, "tokens": toks[:head], "want": list(range(head))})
            elif head <= pos < len(toks):
                entries.append({"id": rid, "tokens": [toks[pos]], "want": [0]})
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": []})
    steps[-1]["end"] = ["a"]
    for step in reversed(steps):
        if any(e["id"] == "b" for e in step["entries"]):
            step["end"] = step["end"] + ["b"]
            break
    _, _, cache, runner = make_runner(
        folder, _ops("hip", dtype), block_size=16, num_blocks=schedules.pages_needed(steps, 16), max_requests=2
    )
    cache.poison()
    _compare(schedules.run_schedule(runner, cache, steps), requests, weights, cfg, dtype)


@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("which", ["A", "C"])
def test_layer_outputs_match_plain(tmp_path, which, backend, dtype):
    folder, cfg, weights = make_dir(tmp_path, which)
    toks = random_tokens(31, cfg["vocab"], 8)
    _, _, cache, runner = make_runner(folder, _ops(backend, dtype), block_size=16, num_blocks=4, max_requests=1)
    cache.create_request("a")
    out = runner.step([StepEntry.of("a", toks, [0, 17, 30])], capture_sites=True)
    _, layers = plain.forward(cfg, _f64(weights), toks)
    assert out.site_outputs.shape == (len(cfg["layers"]), 3, cfg["width"])
    want = layers[:, [0, 17, 30]]
    got = out.site_outputs.double().cpu()
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)
        return
    # bfloat16: a row within 6 %, or within 3 times of what rounding alone does to it (a router's close call)
    coarse = plain.forward(cfg, _f64(weights), toks, round_to=torch.bfloat16)[1][:, [0, 17, 30]]
    size = want.pow(2).sum(-1).sqrt()
    rel, alone = (got - want).pow(2).sum(-1).sqrt() / size, (coarse - want).pow(2).sum(-1).sqrt() / size
    assert bool((rel < torch.clamp(3.0 * alone, min=6e-2)).all()), (rel, alone)


@pytest.mark.parametrize("dtype", GPU_CASES)
def test_replayed_steps_equal_plain_steps(tmp_path, dtype):
    """Steps of a model with streams, state slots and routed experts are recorded and replayed; the replays give
    what the unrecorded steps give, bit for bit."""
    folder, cfg, _ = make_dir(tmp_path, "A")
    requests = {"a": random_tokens(90, cfg["vocab"], 1), "b": random_tokens(75, cfg["vocab"], 2)}
    steps = schedules.bulk_then_tail(requests, tail=40)
    results = []
    for use_graphs in (False, True):
        _, _, cache, runner = make_runner(folder, _ops("hip", dtype), block_size=16, num_blocks=16, max_requests=2)
        runner.use_graphs = use_graphs
        results.append(schedules.run_schedule(runner, cache, steps))
    plain_steps, replayed = results
    assert plain_steps.keys() == replayed.keys()
    for key in plain_steps:
        assert torch.equal(plain_steps[key], replayed[key]), key


# ---- generation through the engine ------------------------------------------------------------------------

@pytest.mark.parametrize("backend,dtype", CASES)
@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_generation_through_the_engine(tmp_path, which, backend, dtype):
    folder, cfg, weights = make_dir(tmp_path, which)
    ops = _ops(backend, dtype)
    engine = ContinuousBatchEngine.from_model_dir(
        folder, dtype=ops.dtype, ops=ops, block_size=BLOCK[which], num_blocks=40, max_running_requests=3,
        max_batch_tokens=24,
    )
    prompts = [random_tokens(n, cfg["vocab"], 9 + n) for n in (5, 30, 1, 17)]
    outs = engine.generate(prompts, max_new_tokens=24)  # long enough to pass page borders while decoding
    w64 = _f64(weights)
    for prompt, tokens in zip(prompts, outs):
        assert len(tokens) == 24
        seq = list(prompt)
        for i, tok in enumerate(tokens):
            logits = plain.forward(cfg, w64, seq)[0][-1]
            best = int(torch.argmax(logits))
            if tok != best:
                # only rounding may choose between two nearly equal logits, and only in bfloat16
                assert dtype == torch.bfloat16, f"token {i}: {tok} != {best}"
                assert float(logits[best] - logits[tok]) < 6e-2 * float(logits.abs().max())
                break
            seq.append(tok)


# ---- the command line and the replay program --------------------------------------------------------------

def test_preset_and_random_model_writer(tmp_path):
    from helpers import read_weights
    from mini_llm_runtime_amd import cli
    from mini_llm_runtime_amd.config.presets import preset_names

    assert "pepulix-tiny" in preset_names()
    assert cli.main(["random-model", "--config", "pepulix-tiny", "--seed", "2", "--out", str(tmp_path / "m")]) == 0
    cfg, w = read_weights(tmp_path / "m")
    assert cfg["architecture"] == "Pepulix" and w["embed"].shape == (320, 96) and "head" not in w
    assert w["l0.hc1.mix"].shape == (2, 2) and w["l1.mix.vmix"].shape == () and w["l2.mlp.e3.down"].shape == (96, 48)
    assert w["l2.mlp.router"].shape == (6, 96) and "l3.norm2" not in w
    logits, layers = plain.forward(cfg, _f64(w), [1, 2, 3])  # the plain implementation reads the same folder
    assert logits.shape == (3, 320) and layers.shape == (4, 3, 96) and torch.isfinite(logits).all()


@pytest.mark.gpu
def test_generate_command_and_trace_replay(tmp_path, gpu_device):
    import subprocess
    import sys

    import numpy as np

    folder, cfg, weights = make_dir(tmp_path, "A")
    w64 = _f64(weights)
    prompt = random_tokens(21, cfg["vocab"], 4)
    proc = subprocess.run(
        [sys.executable, "-m", "mini_llm_runtime_amd.cli", "generate", "--model", str(folder), "--dtype", "float32",
         "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "5"],
        cwd=ROOT, capture_output=True, text=True, timeout=300,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads(proc.stdout.strip().splitlines()[-1])
    seq = list(prompt)
    for tok in out["generated_token_ids"]:
        assert tok == int(torch.argmax(plain.forward(cfg, w64, seq)[0][-1]))
        seq.append(tok)
    # the replay program: requests in portions beside each other, slots and pages used again
    toks = {"a": random_tokens(40, cfg["vocab"], 5), "b": random_tokens(27, cfg["vocab"], 6), "c": random_tokens(33, cfg["vocab"], 7)}
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": toks["a"][:25], "want": [0, 24]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks["a"][25:27], "want": [1]}, {"id": "b", "tokens": toks["b"], "want": [26]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": toks["a"][27:], "want": [12]}, {"id": "c", "tokens": toks["c"][:32], "want": []}], "end": ["a"]},
        {"step": 3, "entries": [{"id": "c", "tokens": toks["c"][32:], "want": [0]}], "end": ["c"]},
    ]
    for dtype, bound in (("float32", 1e-4), ("bfloat16", 6e-2)):
        proc = subprocess.run(
            [str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype, "--out", str(tmp_path / dtype),
             "--max-tokens", "128", "--max-live", "2"],
            input="".join(json.dumps(s) + "\n" for s in steps), cwd=ROOT, capture_output=True, text=True, timeout=300,
        )
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
        wanted = {0: [("a", 0), ("a", 24)], 1: [("a", 26), ("b", 26)], 2: [("a", 39)], 3: [("c", 32)]}
        for step, rows in wanted.items():
            got = torch.from_numpy(np.fromfile(tmp_path / dtype / f"{step}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"]))
            for row, (rid, pos) in zip(got, rows):
                ref = plain.forward(cfg, w64, toks[rid][: pos + 1])[0][-1]
                rel = float((row.double() - ref).pow(2).sum().sqrt() / ref.pow(2).sum().sqrt())
                if dtype == "bfloat16" and rel >= bound:  # held against what rounding alone does to this row
                    coarse = plain.forward(cfg, w64, toks[rid][: pos + 1], round_to=torch.bfloat16)[0][-1]
                    bound = max(bound, 3.0 * float((coarse - ref).pow(2).sum().sqrt() / ref.pow(2).sum().sqrt()))
                assert rel < bound, (dtype, step, rid, pos, rel)
