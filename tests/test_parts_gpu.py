"""Each part alone against the plain functions, and a toy architecture defined here: a mixer with state
of its own, a feed-forward with routing and another position encoding are registered, built from a
configuration, loaded from a model folder and stepped without a change to the framework's files; its plan
names a layer twice and lets a layer read another layer's cache."""
import os

import numpy as np
import pytest
import torch

import helpers as H
import plain_llama as P

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda:0")
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def runtime(dtype, max_positions=256):
    from allpaca_amd.parts import Runtime
    return Runtime(DEV, TORCH[dtype], max_positions)


def f64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def tol(dtype):
    """An output computed in 32-bit from exact inputs: float32 rounding noise, plus, if it is stored in bfloat16,
    one rounding to nearest (half a unit of an 8-bit significand: 2^-8 of the value at most)."""
    return dict(atol=2e-5, rtol=1e-5) if dtype == "float32" else dict(atol=2e-5, rtol=2.0 ** -8 * 1.01)


def assert_part_close(got, exact, stored, dtype, what=""):
    """float32: close to the exact result.  bfloat16: off from the exact result by at most 2.5 times what
    rounding the stored activations to bfloat16 costs by itself (`stored`: the plain result with those roundings
    and exact arithmetic otherwise), plus one rounding of a bfloat16 output."""
    got, exact = np.asarray(got, np.float64), np.asarray(exact, np.float64)
    d = np.abs(got - exact).max()
    if dtype == "float32":
        assert d <= 2e-5 * max(1.0, np.abs(exact).max()), f"{what}: max diff {d:.3e}"
    else:
        lim = 2.5 * np.abs(np.asarray(stored, np.float64) - exact).max() + 2.0 ** -8 * np.abs(exact).max()
        assert d <= lim, f"{what}: max diff {d:.3e}, limit {lim:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_part(dtype):
    from allpaca_amd.parts import NORMS, PartSpec, build_part
    part = build_part(NORMS, PartSpec("rmsnorm", dict(size=120, eps=3e-6)))
    assert part.param_specs()["weight"].shape == (120,) and part.param_specs()["weight"].store == "float32"
    w = 1 + 0.1 * rnd(120, seed=1)
    part.bind({"weight": w}, runtime(dtype))
    x = rnd(9, 120, seed=2, scale=2.0).to(DEV)
    out = torch.empty(9, 120, dtype=TORCH[dtype], device=DEV)
    part.forward(x, out)
    assert np.allclose(f64(out), P.rms_norm(f64(x), f64(w), 3e-6), **tol(dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rotary_part(dtype):
    from allpaca_amd.parts import POSITION_ENCODINGS, PartSpec, build_part
    scaling = dict(rope_type="llama3", factor=4.0, low_freq_factor=1.0, high_freq_factor=2.0,
                   original_max_position_embeddings=32)
    part = build_part(POSITION_ENCODINGS, PartSpec("rope", dict(head_dim=48, theta=250000.0, scaling=scaling)))
    part.bind({}, runtime(dtype))
    rot, table = part.fused()
    assert rot == 48 and tuple(table.shape) == (256, 2, 24)
    inv = P.rope_inv_freq(48, 250000.0, scaling)
    assert np.allclose(f64(table[100, 0]), np.cos(100 * inv), atol=1e-7)   # angles made in 64-bit, rounded once
    H_, Hk = 3, 1
    qk = rnd(5, (H_ + Hk) * 48, seed=3).to(TORCH[dtype])
    dev = qk.clone().to(DEV)
    pos = [0, 7, 8, 200, 255]
    part.apply(dev, 0, H_ * 48, H_, Hk, 48, torch.tensor(pos, dtype=torch.int32, device=DEV))
    want = P.rope_neox(f64(qk).reshape(5, H_ + Hk, 48), pos, inv).reshape(5, -1)
    assert np.allclose(f64(dev), want, **tol(dtype))
    assert torch.equal(dev[0].cpu(), qk[0])      # position 0 is the identity


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_swiglu_part_and_head(dtype):
    from allpaca_amd.parts import FEED_FORWARDS, HEADS, EMBEDDINGS, PartSpec, build_part
    rt = runtime(dtype)
    part = build_part(FEED_FORWARDS, PartSpec("swiglu", dict(hidden_size=72, intermediate_size=200)))
    w = {"gate_proj.weight": rnd(200, 72, seed=1, scale=0.2).to(TORCH[dtype]),
         "up_proj.weight": rnd(200, 72, seed=2, scale=0.2).to(TORCH[dtype]),
         "down_proj.weight": rnd(72, 200, seed=3, scale=0.2).to(TORCH[dtype])}
    assert {k: v.shape for k, v in part.param_specs().items()} == {k: tuple(v.shape) for k, v in w.items()}
    part.bind(w, rt)
    h = rnd(70, 72, seed=4).to(TORCH[dtype]).to(DEV)
    res = rnd(70, 72, seed=5).to(DEV)
    before = f64(res)
    part.forward_add(h, None, res)
    wg, wu, wd = f64(w["gate_proj.weight"]), f64(w["up_proj.weight"]), f64(w["down_proj.weight"])
    act = P.silu(f64(h) @ wg.T) * (f64(h) @ wu.T)
    assert_part_close(f64(res), before + act @ wd.T, before + P.round_bf16(act) @ wd.T, dtype, "swiglu part")
    emb = build_part(EMBEDDINGS, PartSpec("token_table", dict(vocab_size=515, hidden_size=72)))
    table = rnd(515, 72, seed=6).to(TORCH[dtype])
    emb.bind({"weight": table}, rt)
    x = torch.empty(4, 72, device=DEV)
    emb.forward(torch.tensor([0, 514, 7, 7], dtype=torch.int32, device=DEV), x)
    assert torch.equal(x.cpu(), table.float()[[0, 514, 7, 7]])
    head = build_part(HEADS, PartSpec("linear", dict(vocab_size=515, hidden_size=72, tied=True)))
    assert head.param_specs() == {}
    head.bind({}, rt, shared=emb.weight)
    logits = torch.empty(4, 515, device=DEV)
    hh = rnd(4, 72, seed=7).to(TORCH[dtype]).to(DEV)
    head.forward(hh, logits)
    assert_part_close(f64(logits), f64(hh) @ f64(table).T, f64(hh) @ f64(table).T, "float32", "head")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [None, 6])
def test_attention_part_alone(dtype, window):
    """The attention part with a cache manager of its own: two requests, a portion then single rows, compared
    with the plain attention over the whole sequences (with a window too, which llama does not use)."""
    from allpaca_amd.cache import CacheManager, CacheStorage
    from allpaca_amd.engine.batch import Entry, pack_step
    from allpaca_amd.parts import MIXERS, PartSpec, PlanEntry, build_part
    D, Hh, Hk, d = 40, 5, 1, 16
    part = build_part(MIXERS, PartSpec("attention", dict(hidden_size=D, num_heads=Hh, num_kv_heads=Hk, head_dim=d,
                                                         window=window,
                                                         position=PartSpec("rope", dict(head_dim=d, theta=10000.0)))))
    w = {n: rnd(*ps.shape, seed=i, scale=0.4).to(TORCH[dtype]) for i, (n, ps) in enumerate(part.param_specs().items())}
    part.bind(w, runtime(dtype, 64))
    need = part.cache_need()
    assert (need.kv_heads, need.head_dim, need.window) == (Hk, d, window)
    cm = CacheManager([need], 4, 40, 4)
    st = CacheStorage(cm, TORCH[dtype], DEV)
    view = st.views([PlanEntry(0)])[0]
    lens = {"a": 23, "b": 9}
    hs = {k: rnd(n, D, seed=10 + i).to(TORCH[dtype]) for i, (k, n) in enumerate(lens.items())}
    got = {k: [] for k in lens}
    cuts = [[("a", 10), ("b", 2)], [("a", 1), ("b", 1)], [("a", 1)], [("b", 6), ("a", 11)]]
    at = {k: 0 for k in lens}
    for k in lens:
        cm.admit(k)
    for cut in cuts:
        entries = [Entry(k, [0] * n, []) for k, n in cut]
        for k, n in cut:
            cm.reserve(k, n)
        step = pack_step(entries, [cm.length(k) for k, _ in cut], [cm.slot_of(k) for k, _ in cut],
                         [[cm.block_table(k, 0) for k, _ in cut]], DEV, [st.dummy_page(0)])
        view.block_table = step.block_tables[0]
        h = torch.cat([hs[k][at[k]:at[k] + n] for k, n in cut]).to(DEV)
        res = torch.zeros(h.shape[0], D, device=DEV)
        part.forward_add(h, step, view, res)
        r0 = 0
        for k, n in cut:
            got[k].append(f64(res[r0:r0 + n]))
            r0 += n
            at[k] += n
            cm.commit(k, n)
        cm.check()
    inv = P.rope_inv_freq(d, 10000.0)
    for k, n in lens.items():
        h64 = f64(hs[k])
        def plain(st):
            q = st(P.rope_neox(st(h64 @ f64(w["q_proj.weight"]).T).reshape(n, Hh, d), range(n), inv))
            kk = st(P.rope_neox(st(h64 @ f64(w["k_proj.weight"]).T).reshape(n, Hk, d), range(n), inv))
            v = st(h64 @ f64(w["v_proj.weight"]).T).reshape(n, Hk, d)
            return st(P.attention(q, kk, v, Hh, Hk, window=window).reshape(n, Hh * d)) @ f64(w["o_proj.weight"]).T
        assert_part_close(np.concatenate(got[k]), plain(lambda z: z), plain(P.round_bf16), dtype, f"attention part {k}")
    if window:
        assert -1 in cm.block_table("a", 0)      # pages that the window has passed were given back


# --------------------------------------------------------------------------------------------------
# a toy architecture, defined here and nowhere in the framework
# --------------------------------------------------------------------------------------------------
def register_toy():
    from allpaca_amd.models import ARCHITECTURES, Architecture
    from allpaca_amd.parts import (FEED_FORWARDS, MIXERS, POSITION_ENCODINGS, BlockSpec, FeedForward, FixedState,
                                   Mixer, ModelSpec, ParamSpec, PartSpec, PlanEntry, PositionEncoding)
    from allpaca_amd.kernels import ops

    if "toy_decay" in MIXERS:
        return

    @MIXERS.register("toy_decay")
    class DecayMixer(Mixer):
        """State s of the request (a vector per layer): s <- decay * s + h_row, row after row; out = s W^T."""

        def __init__(self, hidden_size, decay):
            self.D, self.decay = hidden_size, decay

        def param_specs(self):
            return {"mix.weight": ParamSpec((self.D, self.D), store="float32")}

        def cache_need(self):
            return FixedState((self.D,), "float32")

        def bind(self, tensors, rt):
            self.rt = rt
            self.w = tensors["mix.weight"].to(rt.device, torch.float32)

        def forward(self, h, step, cache):
            out = torch.empty(h.shape[0], self.D, dtype=torch.float32, device=h.device)
            hf = h.float()
            for r0, n, slot in zip(step.host_row0, step.host_rows, step.host_slots):
                s = cache.state[slot].clone()
                for r in range(r0, r0 + n):
                    s = self.decay * s + hf[r]
                    out[r] = s @ self.w.T
                if cache.writes:
                    cache.state[slot] = s
            return out

    @FEED_FORWARDS.register("toy_routed")
    class RoutedFeedForward(FeedForward):
        """Two experts (plain matrices); a row goes to the expert with the larger router logit (first wins a tie),
        the router logits in 32-bit."""

        def __init__(self, hidden_size):
            self.D = hidden_size

        def param_specs(self):
            return {"router.weight": ParamSpec((2, self.D), store="float32"),
                    "experts.0.weight": ParamSpec((self.D, self.D)), "experts.1.weight": ParamSpec((self.D, self.D))}

        def bind(self, tensors, rt):
            self.rt = rt
            self.router = tensors["router.weight"].to(rt.device, torch.float32)
            self.experts = [tensors[f"experts.{i}.weight"].to(rt.device).contiguous() for i in range(2)]

        def forward_add(self, h, step, residual):
            logits = h.float() @ self.router.T
            choice = (logits[:, 1] > logits[:, 0]).to(torch.int32)
            for e in range(2):
                rows = torch.nonzero(choice == e).flatten().to(torch.int32)
                if rows.numel() == 0:
                    continue
                he = torch.empty(rows.numel(), self.D, dtype=h.dtype, device=h.device)
                ops.gather_rows(h, rows, he)
                ye = torch.empty(rows.numel(), self.D, dtype=torch.float32, device=h.device)
                ops.linear(he, self.experts[e], ye)             # the engine's own matrix product
                residual.index_add_(0, rows.long(), ye)

    @POSITION_ENCODINGS.register("toy_scale")
    class ScaleEncoding(PositionEncoding):
        """Not a rotation: q and k are multiplied by 1 + gain * position / 100 before k is cached."""

        def __init__(self, gain):
            self.gain = gain

        def fused(self):
            return None

        def apply(self, qkv, q_off, k_off, n_heads, n_kv_heads, head_dim, positions):
            f = (1.0 + self.gain * positions.float() / 100.0).unsqueeze(1)
            width = (n_heads + n_kv_heads) * head_dim
            qkv[:, q_off:q_off + width] = (qkv[:, q_off:q_off + width].float() * f).to(qkv.dtype)

    def read_config(d):
        return dict(d)

    def describe(c):
        D, V = c["hidden_size"], c["vocab_size"]
        norm = dict(size=D, eps=c["eps"])
        attn = lambda pos: PartSpec("attention", dict(hidden_size=D, num_heads=c["heads"], num_kv_heads=c["kv_heads"],
                                                      head_dim=c["head_dim"], position=pos), "attn.")
        blocks = []
        for l, kind in enumerate(c["layers"]):
            if kind == "rope_attn":
                mixer = attn(PartSpec("rope", dict(head_dim=c["head_dim"], theta=c["theta"])))
                ffn = PartSpec("swiglu", dict(hidden_size=D, intermediate_size=c["ffn"]), "mlp.")
            elif kind == "scale_attn":
                mixer = attn(PartSpec("toy_scale", dict(gain=c["gain"])))
                ffn = PartSpec("toy_routed", dict(hidden_size=D), "moe.")
            else:
                mixer = PartSpec("toy_decay", dict(hidden_size=D, decay=c["decay"]), "decay.")
                ffn = PartSpec("toy_routed", dict(hidden_size=D), "moe.")
            blocks.append(BlockSpec("pre_norm", {"mixer_norm": PartSpec("rmsnorm", norm, "norm1."), "mixer": mixer,
                                                 "ffn_norm": PartSpec("rmsnorm", norm, "norm2."), "ffn": ffn},
                                    f"toy.layers.{l}."))
        plan = [PlanEntry(b, co) for b, co in c["plan"]]
        return ModelSpec(D, V, c["max_positions"], PartSpec("token_table", dict(vocab_size=V, hidden_size=D), "toy.embed."),
                         blocks, plan, PartSpec("rmsnorm", norm, "toy.norm."),
                         PartSpec("linear", dict(vocab_size=V, hidden_size=D, tied=False), "toy.head."))

    ARCHITECTURES.register("ToyForCausalLM", Architecture("toy", read_config, describe))


TOY = dict(architectures=["ToyForCausalLM"], vocab_size=90, hidden_size=48, heads=3, kv_heads=1, head_dim=16, ffn=56,
           eps=1e-5, theta=10000.0, gain=0.7, decay=0.5, max_positions=128,
           layers=["rope_attn", "decay", "scale_attn"],
           # block 0, block 1 (state), block 2, then block 1 again with a state of its own, then block 0 again
           # reading the cache that its first run wrote
           plan=[[0, None], [1, None], [2, None], [1, None], [0, 0]])


def toy_plain(cfg, w, tokens):
    """The toy model, whole sequence, float64."""
    T, D = len(tokens), cfg["hidden_size"]
    Hh, Hk, d = cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    x = np.asarray(w["toy.embed.weight"], np.float64)[tokens]
    pos = np.arange(T)
    kv_of = {}
    for i, (b, cache_of) in enumerate(cfg["plan"]):
        p = f"toy.layers.{b}."
        kind = cfg["layers"][b]
        h = P.rms_norm(x, w[p + "norm1.weight"], cfg["eps"])
        if kind == "decay":
            s = np.zeros(D)
            out = np.zeros((T, D))
            for t in range(T):
                s = cfg["decay"] * s + h[t]
                out[t] = s @ w[p + "decay.mix.weight"].T
            x = x + out
        else:
            q = P.linear(h, w[p + "attn.q_proj.weight"]).reshape(T, Hh, d)
            k = P.linear(h, w[p + "attn.k_proj.weight"]).reshape(T, Hk, d)
            v = P.linear(h, w[p + "attn.v_proj.weight"]).reshape(T, Hk, d)
            if kind == "rope_attn":
                inv = P.rope_inv_freq(d, cfg["theta"])
                q, k = P.rope_neox(q, pos, inv), P.rope_neox(k, pos, inv)
            else:
                f = (1.0 + cfg["gain"] * pos / 100.0)[:, None, None]
                q, k = q * f, k * f
            if cache_of is None:
                kv_of[i] = (k, v)
            else:
                k, v = kv_of[cache_of]
            o = P.attention(q, k, v, Hh, Hk).reshape(T, Hh * d)
            x = x + P.linear(o, w[p + "attn.o_proj.weight"])
        h = P.rms_norm(x, w[p + "norm2.weight"], cfg["eps"])
        if kind == "rope_attn":
            x = x + P.swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        else:
            lg = h @ w[p + "moe.router.weight"].T
            e = (lg[:, 1] > lg[:, 0]).astype(int)
            y = np.stack([h[t] @ w[p + f"moe.experts.{e[t]}.weight"].T for t in range(T)])
            x = x + y
    return P.rms_norm(x, w["toy.norm.weight"], cfg["eps"]) @ w["toy.head.weight"].T


def test_toy_architecture_registers_builds_and_steps():
    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    from allpaca_amd.weights import write_model_folder
    register_toy()
    folder = os.path.join(H.tmp_root(), "toy_model")
    write_model_folder(folder, TOY, seed=4, dtype=torch.float32, std=0.25, norm_std=0.1)
    cfg, model = load_model(folder, torch.float32, "cuda:0")
    needs = model.cache_needs()
    assert [type(n).__name__ for n in needs] == ["PagedKV", "FixedState", "PagedKV", "FixedState", "NoneType"]
    runner = ModelRunner(model, 4, 40, 3, use_graphs=True)
    assert not runner.use_graphs                      # the toy mixer plans on the host: no graph replay
    assert len(runner.cache.paged_groups) == 1 and runner.cache.paged_groups[0].entries == [0, 2]
    assert [g.entries for g in runner.cache.state_groups] == [[1, 3]]
    _, w = P.read_model_folder(folder)
    toks = {k: H.random_tokens(90, n, seed=i) for i, (k, n) in enumerate([("a", 40), ("b", 17), ("c", 29)])}
    want = {k: toy_plain(TOY, w, t) for k, t in toks.items()}
    # whole
    for k, t in toks.items():
        runner.admit(k)
        got = runner.step([Entry(k, t, list(range(len(t))))]).cpu().numpy()
        runner.release(k)
        assert np.abs(got - want[k]).max() < 1e-4, k
    # portions and single tokens of a and b mixed; c joins later and takes the slot and pages a left behind
    got = {k: [] for k in toks}
    plan = [[("a", 7), ("b", 2)], [("a", 1), ("b", 5)], [("a", 30)], [("b", 1), ("a", 2)], [("b", 9)]]
    for k in ("a", "b"):
        runner.admit(k)
    at = {k: 0 for k in toks}
    def run(batch):
        lg = runner.step([Entry(k, toks[k][at[k]:at[k] + n], list(range(n))) for k, n in batch]).cpu().numpy()
        r = 0
        for k, n in batch:
            got[k].append(lg[r:r + n])
            r += n
            at[k] += n
    for batch in plan:
        run(batch)
    slot_a = runner.cache.slot_of("a")
    runner.release("a")
    runner.admit("c")
    assert runner.cache.slot_of("c") == slot_a                         # the slot is recycled ...
    assert float(runner.storage.state[0][:, slot_a].abs().max()) == 0.0  # ... and reads zeros
    run([("c", 13)])
    run([("c", 1)])
    run([("c", 15)])
    for k in toks:
        assert np.abs(np.concatenate(got[k]) - want[k]).max() < 1e-4, k
    runner.cache.check()


# --------------------------------------------------------------------------------------------------
# a second toy architecture: a cache need of the mixer's own (one latent vector per position, no values, 32-bit
# whatever the run's cache type), a position encoding over two axes, and a feed-forward that plans on the host
# beside a mixer that does not
# --------------------------------------------------------------------------------------------------
def register_toy2():
    from dataclasses import dataclass
    from typing import Optional

    from allpaca_amd.models import ARCHITECTURES, Architecture
    from allpaca_amd.parts import (MIXERS, POSITION_ENCODINGS, BlockSpec, Mixer, ModelSpec, ParamSpec, PartSpec,
                                   PlanEntry, PositionEncoding)
    register_toy()
    if "toy_latent" in MIXERS:
        return

    @dataclass(frozen=True)
    class LatentPages:
        """One vector of `width` numbers per position, in pages, always float32."""
        width: int
        window: Optional[int] = None
        kind = "pages"
        dtype = "float32"

        def page_shape(self, page_tokens):
            return (page_tokens, self.width)

    @MIXERS.register("toy_latent")
    class LatentMixer(Mixer):
        """c_t = h_t Wd^T is cached (nothing else); out_t = mean(c_0 .. c_t) Wu^T."""

        def __init__(self, hidden_size, width):
            self.D, self.r = hidden_size, width

        def param_specs(self):
            return {"down.weight": ParamSpec((self.r, self.D), store="float32"),
                    "up.weight": ParamSpec((self.D, self.r), store="float32")}

        def cache_need(self):
            return LatentPages(self.r)

        def bind(self, tensors, rt):
            self.rt = rt
            self.wd = tensors["down.weight"].to(rt.device, torch.float32)
            self.wu = tensors["up.weight"].to(rt.device, torch.float32)

        def forward(self, h, step, cache):
            Pg = cache.page_tokens
            assert tuple(cache.kv.shape[1:]) == (Pg, self.r) and cache.kv.dtype == torch.float32
            out = torch.empty(h.shape[0], self.D, dtype=torch.float32, device=h.device)
            for s, (r0, n, p0) in enumerate(zip(step.host_row0, step.host_rows, step.host_pos0)):
                c = h[r0:r0 + n].float() @ self.wd.T
                bt = cache.block_table[s].long()
                pos = torch.arange(p0, p0 + n, device=h.device)
                if cache.writes:
                    cache.kv[bt[pos // Pg], pos % Pg] = c
                every = torch.arange(0, p0 + n, device=h.device)
                lat = cache.kv[bt[every // Pg], every % Pg]
                mean = lat.cumsum(0)[p0:] / (pos + 1).unsqueeze(1).float()
                out[r0:r0 + n] = mean @ self.wu.T
            return out

    @POSITION_ENCODINGS.register("toy_axes")
    class TwoAxes(PositionEncoding):
        """q and k are multiplied by 1 + gain * (a0 + 2 a1) / 100 for a token at (a0, a1)."""

        def __init__(self, gain):
            self.gain = gain

        def fused(self):
            return None

        def apply(self, qkv, q_off, k_off, n_heads, n_kv_heads, head_dim, positions):
            assert positions.dim() == 2 and positions.shape[1] == 2
            f = (1.0 + self.gain * (positions[:, 0] + 2 * positions[:, 1]).float() / 100.0).unsqueeze(1)
            width = (n_heads + n_kv_heads) * head_dim
            qkv[:, q_off:q_off + width] = (qkv[:, q_off:q_off + width].float() * f).to(qkv.dtype)

    def describe(c):
        D, V = c["hidden_size"], c["vocab_size"]
        norm = dict(size=D, eps=c["eps"])
        attn = lambda pos: PartSpec("attention", dict(hidden_size=D, num_heads=c["heads"], num_kv_heads=c["kv_heads"],
                                                      head_dim=c["head_dim"], position=pos), "attn.")
        blocks = []
        for l, kind in enumerate(c["layers"]):
            if kind == "latent":
                mixer = PartSpec("toy_latent", dict(hidden_size=D, width=c["latent"]), "latent.")
                ffn = PartSpec("swiglu", dict(hidden_size=D, intermediate_size=c["ffn"]), "mlp.")
            elif kind == "axes_attn_routed":
                mixer = attn(PartSpec("toy_axes", dict(gain=c["gain"])))
                ffn = PartSpec("toy_routed", dict(hidden_size=D), "moe.")
            else:
                mixer = attn(PartSpec("rope", dict(head_dim=c["head_dim"], theta=c["theta"])))
                ffn = PartSpec("toy_routed", dict(hidden_size=D), "moe.")
            blocks.append(BlockSpec("pre_norm", {"mixer_norm": PartSpec("rmsnorm", norm, "norm1."), "mixer": mixer,
                                                 "ffn_norm": PartSpec("rmsnorm", norm, "norm2."), "ffn": ffn},
                                    f"toy.layers.{l}."))
        return ModelSpec(D, V, c["max_positions"], PartSpec("token_table", dict(vocab_size=V, hidden_size=D), "toy.embed."),
                         blocks, [PlanEntry(b) for b in range(len(blocks))], PartSpec("rmsnorm", norm, "toy.norm."),
                         PartSpec("linear", dict(vocab_size=V, hidden_size=D, tied=False), "toy.head."),
                         position_axes=c["axes"])

    ARCHITECTURES.register("Toy2ForCausalLM", Architecture("toy2", dict, describe))


TOY2 = dict(architectures=["Toy2ForCausalLM"], vocab_size=70, hidden_size=32, heads=2, kv_heads=2, head_dim=16, ffn=40,
            latent=5, eps=1e-5, theta=10000.0, gain=0.6, max_positions=96, axes=2, layers=["latent", "axes_attn_routed"])


def toy2_plain(cfg, w, tokens, axis1=None):
    """The second toy model, whole sequence, float64.  `axis1`: the tokens' places on the second axis."""
    T = len(tokens)
    Hh, Hk, d = cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    x = np.asarray(w["toy.embed.weight"], np.float64)[tokens]
    pos = np.arange(T)
    a1 = pos if axis1 is None else np.asarray(axis1)
    for l, kind in enumerate(cfg["layers"]):
        p = f"toy.layers.{l}."
        h = P.rms_norm(x, w[p + "norm1.weight"], cfg["eps"])
        if kind == "latent":
            c = h @ w[p + "latent.down.weight"].T
            mean = np.cumsum(c, axis=0) / (pos + 1)[:, None]
            x = x + mean @ w[p + "latent.up.weight"].T
        else:
            q = P.linear(h, w[p + "attn.q_proj.weight"]).reshape(T, Hh, d)
            k = P.linear(h, w[p + "attn.k_proj.weight"]).reshape(T, Hk, d)
            v = P.linear(h, w[p + "attn.v_proj.weight"]).reshape(T, Hk, d)
            if kind == "axes_attn_routed":
                f = (1.0 + cfg["gain"] * (pos + 2 * a1) / 100.0)[:, None, None]
                q, k = q * f, k * f
            else:
                inv = P.rope_inv_freq(d, cfg["theta"])
                q, k = P.rope_neox(q, pos, inv), P.rope_neox(k, pos, inv)
            x = x + P.linear(P.attention(q, k, v, Hh, Hk).reshape(T, Hh * d), w[p + "attn.o_proj.weight"])
        h = P.rms_norm(x, w[p + "norm2.weight"], cfg["eps"])
        if kind == "latent":
            x = x + P.swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        else:
            lg = h @ w[p + "moe.router.weight"].T
            e = (lg[:, 1] > lg[:, 0]).astype(int)
            x = x + np.stack([h[t] @ w[p + f"moe.experts.{e[t]}.weight"].T for t in range(T)])
    return P.rms_norm(x, w["toy.norm.weight"], cfg["eps"]) @ w["toy.head.weight"].T


def test_a_cache_need_of_the_mixers_own_and_positions_on_two_axes():
    """Registered here, with zero edits to the framework: pages that hold one 32-bit vector per position (no values, not
    the run's cache type) in a group of their own beside a group of keys and values, and a position encoding that
    reads two axes (given per request, or the token's place on both)."""
    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    from allpaca_amd.weights import write_model_folder
    register_toy2()
    folder = os.path.join(H.tmp_root(), "toy2_model")
    write_model_folder(folder, TOY2, seed=6, dtype=torch.float32, std=0.25, norm_std=0.1)
    cfg, model = load_model(folder, torch.float32, "cuda:0")
    runner = ModelRunner(model, 4, 30, 3, use_graphs=True)
    assert not runner.use_graphs and runner.position_axes == 2
    kinds = [type(g.need).__name__ for g in runner.cache.paged_groups]
    assert kinds == ["LatentPages", "PagedKV"]
    assert tuple(runner.storage.paged[0].shape) == (1, 31, 4, 5) and runner.storage.paged[0].dtype == torch.float32
    _, w = P.read_model_folder(folder)
    toks = {"a": H.random_tokens(70, 37, seed=1), "b": H.random_tokens(70, 12, seed=2)}
    axis1 = {"a": None, "b": [(7 * i) % 5 for i in range(12)]}
    want = {k: toy2_plain(TOY2, w, t, axis1[k]) for k, t in toks.items()}
    got = {k: [] for k in toks}
    at = {k: 0 for k in toks}
    for k in toks:
        runner.admit(k)
    for batch in ([("a", 9), ("b", 3)], [("a", 1), ("b", 1)], [("a", 20), ("b", 1)], [("b", 7), ("a", 1)], [("a", 6)]):
        entries = []
        for k, n in batch:
            pos = None if axis1[k] is None else [[at[k] + i, axis1[k][at[k] + i]] for i in range(n)]
            entries.append(Entry(k, toks[k][at[k]:at[k] + n], list(range(n)), pos))
        lg = runner.step(entries).cpu().numpy()
        r = 0
        for k, n in batch:
            got[k].append(lg[r:r + n])
            r += n
            at[k] += n
    for k in toks:
        assert np.abs(np.concatenate(got[k]) - want[k]).max() < 1e-4, k
    for k in toks:
        runner.release(k)
    runner.cache.check()
    assert [runner.cache.free_pages(g) for g in range(2)] == [30, 30]


def test_a_feed_forward_that_plans_on_the_host_keeps_the_model_out_of_graphs():
    """Attention (which may be replayed) beside a routed feed-forward that gathers rows per expert on the host: asked
    for graphs, the runner replays none, and decode steps whose rows go to other experts from step to step are right."""
    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    from allpaca_amd.weights import write_model_folder
    register_toy2()
    cfgj = dict(TOY2, layers=["rope_attn_routed", "rope_attn_routed"], axes=1)
    folder = os.path.join(H.tmp_root(), "toy2_routed")
    write_model_folder(folder, cfgj, seed=8, dtype=torch.float32, std=0.25, norm_std=0.1)
    cfg, model = load_model(folder, torch.float32, "cuda:0")
    assert all(b.mixer.graph_safe for b in model.blocks) and not any(b.parts["ffn"].graph_safe for b in model.blocks)
    runner = ModelRunner(model, 4, 30, 3, use_graphs=True)
    assert not runner.use_graphs
    _, w = P.read_model_folder(folder)
    toks = {"a": H.random_tokens(70, 30, seed=3), "b": H.random_tokens(70, 25, seed=4)}
    want = {k: toy2_plain(cfgj, w, t) for k, t in toks.items()}
    for k in toks:
        runner.admit(k)
    runner.step([Entry("a", toks["a"][:10], []), Entry("b", toks["b"][:5], [])])
    for j in range(20):
        lg = runner.step([Entry("a", [toks["a"][10 + j]], [0]), Entry("b", [toks["b"][5 + j]], [0])]).cpu().numpy()
        assert np.abs(lg[0] - want["a"][10 + j]).max() < 1e-4 and np.abs(lg[1] - want["b"][5 + j]).max() < 1e-4, j
    assert runner.graph_replays == 0


# --------------------------------------------------------------------------------------------------
# a third toy architecture: a layer with two parts that each keep something per request (attention heads beside a
# decaying state, in an arrangement of the test's own), and a bias kept in 32-bit that starts at a constant
# --------------------------------------------------------------------------------------------------
def register_toy3():
    from allpaca_amd.models import ARCHITECTURES, Architecture
    from allpaca_amd.parts import (ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS, BlockSpec, FixedState, Mixer, ModelSpec,
                                   ParamSpec, PartSpec, PlanEntry)
    register_toy()
    if "toy_decay_bias" in MIXERS:
        return

    @MIXERS.register("toy_decay_bias")
    class DecayBiasMixer(Mixer):
        """s <- decay * s + h_row + bias, row after row; out = s W^T.  The bias is stored in 32-bit and random weights
        start it at 0.25 (not at 1 + noise, which is what a norm's weight gets)."""

        def __init__(self, hidden_size, decay):
            self.D, self.decay = hidden_size, decay

        def param_specs(self):
            return {"mix.weight": ParamSpec((self.D, self.D), store="float32", init="normal"),
                    "bias": ParamSpec((self.D,), store="float32", init=0.25),
                    "gate": ParamSpec((self.D,), store="float32", init="zeros")}

        def cache_need(self):
            return FixedState((self.D,), "float32")

        def bind(self, tensors, rt):
            self.rt = rt
            self.w = tensors["mix.weight"].to(rt.device, torch.float32)
            self.bias = tensors["bias"].to(rt.device, torch.float32)
            self.gate = tensors["gate"].to(rt.device, torch.float32)

        def forward(self, h, step, cache):
            out = torch.empty(h.shape[0], self.D, dtype=torch.float32, device=h.device)
            hf = h.float()
            for r0, n, slot in zip(step.host_row0, step.host_rows, step.host_slots):
                s = cache.state[slot].clone()
                for r in range(r0, r0 + n):
                    s = self.decay * s + hf[r] + self.bias
                    out[r] = (s * (1.0 + self.gate)) @ self.w.T
                if cache.writes:
                    cache.state[slot] = s
            return out

    @ARRANGEMENTS.register("toy_two_mixers")
    class TwoMixers:
        """x += attention(norm(x)) + recurrent(norm(x)); x += ffn(norm2(x)): two parts with a cache of their own."""
        registries = {"norm": NORMS, "mixer": MIXERS, "recurrent": MIXERS, "ffn_norm": NORMS, "ffn": FEED_FORWARDS}

        @staticmethod
        def run(parts, x, step, cache):
            assert set(cache) == {"mixer", "recurrent"}
            rt = parts["mixer"].rt
            h = torch.empty(x.shape, dtype=rt.dtype, device=x.device)
            parts["norm"].forward(x, h)
            parts["mixer"].forward_add(h, step, cache["mixer"], x)
            parts["recurrent"].forward_add(h, step, cache["recurrent"], x)
            h2 = torch.empty(x.shape, dtype=rt.dtype, device=x.device)
            parts["ffn_norm"].forward(x, h2)
            parts["ffn"].forward_add(h2, step, x)

    def describe(c):
        D, V = c["hidden_size"], c["vocab_size"]
        norm = dict(size=D, eps=c["eps"])
        block = BlockSpec("toy_two_mixers", {
            "norm": PartSpec("rmsnorm", norm, "norm1."),
            "mixer": PartSpec("attention", dict(hidden_size=D, num_heads=c["heads"], num_kv_heads=c["kv_heads"],
                                                head_dim=c["head_dim"],
                                                position=PartSpec("rope", dict(head_dim=c["head_dim"], theta=c["theta"]))),
                              "attn."),
            "recurrent": PartSpec("toy_decay_bias", dict(hidden_size=D, decay=c["decay"]), "rec."),
            "ffn_norm": PartSpec("rmsnorm", norm, "norm2."),
            "ffn": PartSpec("swiglu", dict(hidden_size=D, intermediate_size=c["ffn"]), "mlp.")}, "toy3.layers.0.")
        return ModelSpec(D, V, c["max_positions"], PartSpec("token_table", dict(vocab_size=V, hidden_size=D), "toy3.embed."),
                         [block], [PlanEntry(0), PlanEntry(0)], PartSpec("rmsnorm", norm, "toy3.norm."),
                         PartSpec("linear", dict(vocab_size=V, hidden_size=D, tied=False), "toy3.head."))

    ARCHITECTURES.register("Toy3ForCausalLM", Architecture("toy3", dict, describe))


TOY3 = dict(architectures=["Toy3ForCausalLM"], vocab_size=60, hidden_size=32, heads=2, kv_heads=1, head_dim=16, ffn=40,
            eps=1e-5, theta=10000.0, decay=0.6, max_positions=96)


def toy3_plain(cfg, w, tokens):
    T, D = len(tokens), cfg["hidden_size"]
    Hh, Hk, d = cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    x = np.asarray(w["toy3.embed.weight"], np.float64)[tokens]
    p = "toy3.layers.0."
    inv = P.rope_inv_freq(d, cfg["theta"])
    for _ in range(2):      # the block runs twice, each run with caches of its own
        h = P.rms_norm(x, w[p + "norm1.weight"], cfg["eps"])
        q = P.rope_neox(P.linear(h, w[p + "attn.q_proj.weight"]).reshape(T, Hh, d), np.arange(T), inv)
        k = P.rope_neox(P.linear(h, w[p + "attn.k_proj.weight"]).reshape(T, Hk, d), np.arange(T), inv)
        v = P.linear(h, w[p + "attn.v_proj.weight"]).reshape(T, Hk, d)
        att = P.linear(P.attention(q, k, v, Hh, Hk).reshape(T, Hh * d), w[p + "attn.o_proj.weight"])
        s, rec = np.zeros(D), np.zeros((T, D))
        for t in range(T):
            s = cfg["decay"] * s + h[t] + w[p + "rec.bias"]
            rec[t] = (s * (1.0 + w[p + "rec.gate"])) @ w[p + "rec.mix.weight"].T
        x = x + att + rec
        h = P.rms_norm(x, w[p + "norm2.weight"], cfg["eps"])
        x = x + P.swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.rms_norm(x, w["toy3.norm.weight"], cfg["eps"]) @ w["toy3.head.weight"].T


def test_a_layer_with_two_parts_that_keep_a_cache_and_a_bias_in_32_bit():
    """Defined here and nowhere in the framework: a block whose arrangement has two parts with a cache need each
    (pages of keys and values, a state slot) and a 32-bit bias whose random start is a constant of its own."""
    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    from allpaca_amd.weights import write_model_folder
    register_toy3()
    folder = os.path.join(H.tmp_root(), "toy3_model")
    write_model_folder(folder, TOY3, seed=9, dtype=torch.float32, std=0.25, norm_std=0.1)
    _, w = P.read_model_folder(folder)
    p = "toy3.layers.0."
    assert np.all(w[p + "rec.bias"] == 0.25) and np.all(w[p + "rec.gate"] == 0.0)      # ParamSpec.init
    assert abs(float(np.std(w[p + "rec.mix.weight"])) - 0.25) < 0.05 and abs(float(np.mean(w[p + "rec.mix.weight"]))) < 0.05
    assert abs(float(np.mean(w[p + "norm1.weight"])) - 1.0) < 0.1                       # a norm's weight: 1 + noise
    cfg, model = load_model(folder, torch.float32, "cuda:0")
    needs = model.cache_needs()
    assert [sorted(n) for n in needs] == [["mixer", "recurrent"]] * 2
    runner = ModelRunner(model, 4, 40, 3)
    assert runner.native is None                       # the executor does not know this arrangement: walked in Python
    assert runner.cache.paged_groups[0].entries == [(0, "mixer"), (1, "mixer")]
    assert runner.cache.state_groups[0].entries == [(0, "recurrent"), (1, "recurrent")]
    toks = {"a": H.random_tokens(60, 33, seed=1), "b": H.random_tokens(60, 14, seed=2)}
    want = {k: toy3_plain(TOY3, w, t) for k, t in toks.items()}
    got = {k: [] for k in toks}
    at = {k: 0 for k in toks}
    for k in toks:
        runner.admit(k)
    for batch in ([("a", 9), ("b", 3)], [("a", 1), ("b", 1)], [("a", 20), ("b", 1)], [("b", 9), ("a", 1)], [("a", 2)]):
        lg = runner.step([Entry(k, toks[k][at[k]:at[k] + n], list(range(n))) for k, n in batch]).cpu().numpy()
        r = 0
        for k, n in batch:
            got[k].append(lg[r:r + n])
            r += n
            at[k] += n
    for k in toks:
        assert np.abs(np.concatenate(got[k]) - want[k]).max() < 1e-4, k
        runner.release(k)
    runner.cache.check()
