"""The Bimepel design on the GPU against the plain implementation (``plain_bimepel``): every mechanism alone, then
whole models of several shapes through the step function, the cache, captured decode steps and ``generate``.

The tests make their own small configurations and weights.  Sizes are chosen so that nothing is equal that need not
be (key and value sizes of a head, rotated and whole head, heads and kv heads, block sizes of the mask and the
cache's pages), and a far key, a block's edge or a stale state shows in the result instead of drowning in averages.
"""
import json
import os

import pytest
import torch

import helpers
import plain_bimepel as P

pytestmark = pytest.mark.gpu

DTYPES = [("float32", 3e-5), ("bfloat16", 4e-2)]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def _bf16(t):
    return t.to(torch.bfloat16).double()


def _close(got, want, rel, what):
    got, want = got.double().cpu(), want.double()
    assert got.shape == want.shape, f"{what}: {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: not finite"
    scale = max(1e-6, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= rel * scale, f"{what}: max |diff| {err:.3e} > {rel} x {scale:.3e}"


# ---- configurations ---------------------------------------------------------------------------------------------
def attn(heads=6, kv=2, dim=24, vdim=20, dims=8, base=10000.0, scale=0.3, mask=40, scaling=True):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if dims:
        m["rot"] = {"base": base, "dims": dims}
        if scaling:
            m["rot"]["scaling"] = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    if mask:
        m["mask"] = {"size": mask}
    return {"type": "attention", "mixer": m}


def lin(heads=3, dim=12, vdim=20, decay=(0.5, 0.9, 0.99)):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def dense(layer, ff=56, limit=0.8):
    return dict(layer, mlp={"kind": "dense", "ff": ff, "limit": limit})


def moe(layer, ff=24, experts=5, top=2, scale=1.5):
    return dict(layer, mlp={"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}})


def bare(layer):
    return dict(layer, mlp=None)


def config(layers, loop=None, vocab=131, width=48, eps=1e-5):
    c = {"architecture": "Bimepel", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}
    if loop is not None:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


CONFIGS = {
    # both mixers with every feed-forward, a layer without one, two shapes of attention, a loop of two layers run twice
    "mixed": config([dense(attn()), moe(lin()), moe(attn(4, 1, 16, 32, 16, 5e4, 0.2, 70, False), 16, 7, 3, 2.0),
                     bare(lin(2, 20, 8, (0.8, 0.999))), dense(attn(2, 2, 40, 8, 0, mask=0), 40, 2.0)], loop=(1, 3, 2)),
    # one head, one expert of one, no loop, no mask, no scaling: the values that make indices vanish
    "ones": config([moe(attn(1, 1, 16, 16, 16, 100.0, 0.25, 0, False), 8, 1, 1, 1.0), dense(lin(1, 16, 16, (0.9,)), 16, 1.0)],
                   vocab=61, width=16),
    # the whole model as one loop of three passes; masks of one page, of less and of a size that no page shares
    "loop": config([dense(attn(4, 2, 32, 32, 32, 1e6, 0.18, 64)), moe(attn(4, 4, 16, 24, 8, 1e4, 0.25, 17), 32, 4, 4, 0.7),
                    dense(lin(4, 8, 8, (0.3, 0.6, 0.9, 0.97)), 32, 0.5)], loop=(0, 3, 3), vocab=97, width=64),
}


def make_weights(cfg, seed, std=0.3):
    """Random weights by the design's tensor names, rounded to bfloat16 (so that both compute types hold the same
    numbers), as float64.  Lively enough that layers matter: gains around one, routers that spread their choices."""
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.config.registry import lookup

    c = AutoConfig.from_dict(cfg)
    specs = lookup(c.model_type)[1](c).tensor_specs()
    g = torch.Generator().manual_seed(seed)
    w = {}
    for s in specs:
        if s.tied_to is not None:
            continue
        names = [(s.name, s.shape)] if not s.pieces else list(s.pieces)
        for n, shape in names:
            t = torch.randn(shape, generator=g)
            if n.endswith((".norm1", ".norm2", ".norm")) or n == "final.norm":
                t = 1.0 + 0.3 * t
            elif n.endswith(".shift"):
                t = 0.5 + 0.3 * t
            elif n.endswith(".router"):
                t = t * 0.8
            elif n != "embed":
                t = t * std * (48.0 / shape[-1]) ** 0.5
            w[n] = _bf16(t)
    return w


def write_model(folder, cfg, w):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, os.path.join(folder, "model.safetensors"),
              metadata={"format": "pt"})
    return str(folder)


def load(folder, dtype):
    from pytorch_transformers_amd import AutoModelForCausalLM

    return AutoModelForCausalLM.from_pretrained(str(folder), dtype=dtype)


def plain_all(cfg, w, reqs):
    model = P.PlainBimepel(cfg, w)
    return {rid: model.logits(toks).float() for rid, toks in reqs.items()}


# ---- steps for parts that run alone ---------------------------------------------------------------------------------
def _ctx(cache, slots, new_tokens, dtype):
    import numpy as np

    from pytorch_transformers_amd.engine.step import plan_step
    from pytorch_transformers_amd.parts.base import StepContext

    plan = plan_step(cache, slots, [[0] * n for n in new_tokens], "all", 10)
    i32 = lambda a: torch.as_tensor(np.asarray(a), dtype=torch.int32).cuda()
    ctx = StepContext(dtype=dtype, device=torch.device("cuda:0"), n_seqs=plan.n_seqs, n_tokens=plan.n_tokens,
                      token_seq=i32(plan.token_seq), token_pos=i32(plan.token_pos), cu_tokens=i32(plan.cu_tokens),
                      seq_start=i32(plan.starts), seq_slot=i32(plan.slots),
                      block_tables={g: i32(t) for g, t in plan.block_tables.items()}, cache=cache, slots=plan.slots,
                      new_tokens=plan.new_tokens, starts=plan.starts, is_decode=plan.is_decode, max_len=plan.max_len)
    return ctx, plan


def _run_in_cuts(step, groups, dtype, inputs, cuts_per_seq, free_and_again=False):
    """Feed each sequence of ``inputs`` (float64 ``[T, hidden]``) through ``step(x, ctx)`` in the given cuts, all
    sequences of a turn in one step; returns the outputs per sequence.  ``free_and_again``: the whole is run twice
    on one cache, so that the second run's sequences take slots and pages that the first run's gave back."""
    from pytorch_transformers_amd.cache.paged import PagedCache

    cache = PagedCache(groups, 4096, dtype, "cuda:0", max_slots=8)
    for again in range(2 if free_and_again else 1):
        slots = [cache.alloc() for _ in inputs]
        if again:
            slots = slots[::-1]  # and not the slots they had
        at = [0] * len(inputs)
        outs = [[] for _ in inputs]
        for r in range(max(len(c) for c in cuts_per_seq)):
            live = [i for i, c in enumerate(cuts_per_seq) if r < len(c)]
            ns = [cuts_per_seq[i][r] for i in live]
            ctx, plan = _ctx(cache, [slots[i] for i in live], ns, dtype)
            x = torch.cat([inputs[i][at[i]:at[i] + n] for i, n in zip(live, ns)]).to(dtype).cuda()
            y = step(x, ctx)
            cache.commit(plan.slots, plan.new_tokens)
            o = 0
            for i, n in zip(live, ns):
                outs[i].append(y[o:o + n].double().cpu())
                at[i] += n
                o += n
        for s in slots:
            cache.free(s)
        cache.check_consistent()
    return [torch.cat(o) for o in outs]


def _load_part(part, w, dtype):
    from pytorch_transformers_amd.weights.loader import device_dtype_for

    tensors = {}
    for s in part.all_tensor_specs():
        t = w[s.name] if s.name in w else s.assemble([w[n] for n, _ in s.pieces])
        tensors[s.name] = t.to(device_dtype_for(s, dtype)).cuda().contiguous()
    part.load_all(tensors)
    if hasattr(part, "after_load"):
        part.after_load()

    def walk(p):
        if hasattr(p, "to"):
            p.to("cuda:0")
        for c in p.children():
            walk(c)

    walk(part)


def _part_weights(part, seed, std=0.3):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for s in part.all_tensor_specs():
        for n, shape in ([(s.name, s.shape)] if not s.pieces else list(s.pieces)):
            t = torch.randn(shape, generator=g)
            t = 1.0 + 0.3 * t if n.endswith(".norm") else t * (0.5 if len(shape) == 1 else std)
            w[n] = _bf16(t)
    return w


CUTS = [[61], [1] * 9 + [2, 50], [30, 2, 2, 27], [64 - 3, ]]  # whole; token by token, then a rest; portions down to two
# long enough that the recurrence cuts a sequence into chunks that run side by side, beside sequences that are not cut
LONG_CUTS = [[700], [300, 1, 399], [1, 2, 697], [40, 660]]


# ---- each mechanism alone ------------------------------------------------------------------------------------------------
def test_rotation_frequencies_follow_the_ramp():
    from pytorch_transformers_amd.parts.positions import yarn_ramp_frequencies

    for rot in ({"base": 300000.0, "dims": 48, "scaling": {"factor": 3.0, "original": 1024, "fast": 16.0, "slow": 1.0}},
                {"base": 100.0, "dims": 6, "scaling": {"factor": 8.0, "original": 16, "fast": 2.0, "slow": 0.5}},
                {"base": 1e4, "dims": 32, "scaling": {"factor": 3.0, "original": 4096, "fast": 1.0, "slow": 1.0}}):
        sc = rot["scaling"]
        table, mult = yarn_ramp_frequencies(rot["dims"], rot["base"], sc["factor"], sc["original"], sc["fast"], sc["slow"])
        want, want_mult = P.yarn_frequencies(rot)
        assert abs(mult - want_mult) < 1e-12
        assert torch.allclose(table.double(), want, rtol=1e-7, atol=0)
        assert not torch.allclose(table.double(), P.yarn_frequencies({"base": rot["base"], "dims": rot["dims"]})[0], rtol=1e-3)


@pytest.mark.parametrize("dtype,rel", DTYPES)
def test_shifted_norms_carry_the_token_before(dtype, rel):
    """The stream's two norms and the mix with the token before's first norm: inside a step, over a step's edge
    (the state row), at a sequence's first token, with terms to add, in batches and in slots that are used again."""
    from pytorch_transformers_amd import ops
    from pytorch_transformers_amd.engine.spec import CACHE_STATE, CacheGroupSpec

    H, eps, dt = 40, 1e-5, TORCH[dtype]
    w1, w2, mu = _bf16(1 + 0.3 * _rand(H, seed=1)), _bf16(1 + 0.3 * _rand(H, seed=2)), _bf16(0.5 + 0.4 * _rand(H, seed=3))
    base = [_rand(61, H, seed=10 + i).double() for i in range(4)]
    t1 = [_bf16(_rand(61, H, seed=20 + i)) for i in range(4)]
    t2 = [_bf16(_rand(61, H, seed=30 + i)) for i in range(4)]
    group = CacheGroupSpec("shift", CACHE_STATE, 2, state_shape=(H,))
    dev = lambda t: t.float().cuda()
    for terms in (0, 1, 2):
        def step(x, ctx):
            xb = x[:, :H].float().contiguous()
            ts = [x[:, (1 + j) * H:(2 + j) * H].contiguous() for j in range(terms)]
            stream, a, m = ops.shift_norm(xb, ts, dev(w1), dev(w2), dev(mu), eps, ctx.cache.state_layer("shift", 1), ctx, dt)
            return torch.cat([stream, a.float(), m.float()], dim=1)

        packed = [torch.cat([base[i].to(dt).double(), t1[i], t2[i]], dim=1) for i in range(4)]
        outs = _run_in_cuts(step, [group], dt, packed, CUTS, free_and_again=True)
        for i in range(4):
            x = base[i].to(dt).double()
            if terms:
                x = x + (t1[i] + (t2[i] if terms > 1 else 0))
            n1, n2 = P.rms(x, eps) * w1, P.rms(x, eps) * w2
            before = torch.cat([torch.zeros(1, H, dtype=torch.float64), n1[:-1]])
            _close(outs[i][:, :H], x, 1e-6, f"stream {terms} terms, sequence {i}")
            _close(outs[i][:, H:2 * H], P.shift_mix(n1, before, mu), rel, f"shifted norm, {terms} terms, sequence {i}")
            _close(outs[i][:, 2 * H:], n2, rel, f"second norm, {terms} terms, sequence {i}")


def _attention_mixer(hidden, m, eps=1e-5):
    from pytorch_transformers_amd.engine.bimepel import _positions
    from pytorch_transformers_amd.parts import GatedAttentionMixer

    return GatedAttentionMixer("a", hidden, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], eps, _positions(m),
                               chunk=(m.get("mask") or {}).get("size", 0))


def _plain_attention(w, m, x, eps=1e-5):
    kept, out = {}, []
    for pos in range(x.shape[0]):
        out.append(P.attention_token(w, "a", m, eps, x[pos], pos, kept))
    return torch.stack(out)


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("shape", [attn(), attn(4, 1, 16, 32, 16, 5e4, 0.2, 64, False), attn(2, 2, 40, 8, 0, mask=0),
                                   attn(5, 5, 8, 8, 2, 10.0, 0.5, 7), attn(3, 1, 72, 130, 36, 1e4, 0.1, 100)])
def test_attention_mixer_alone(dtype, rel, shape):
    from pytorch_transformers_amd.engine.spec import CACHE_FULL, CacheGroupSpec

    m, hidden, dt = shape["mixer"], 32, TORCH[dtype]
    mixer = _attention_mixer(hidden, m)
    w = _part_weights(mixer, seed=5)
    _load_part(mixer, w, dt)
    group = CacheGroupSpec("kv", CACHE_FULL, 1, mixer.kv_heads, mixer.frame)
    from pytorch_transformers_amd.engine.spec import LayerCall

    call = LayerCall(0, "kv", 0)
    cuts = [[150], [64, 1, 1, 62, 2, 20], [1] * 20 + [130], [63, 2, 85]]
    xs = [_bf16(_rand(150, hidden, seed=40 + i)) for i in range(4)]
    outs = _run_in_cuts(lambda x, ctx: mixer.forward(x, ctx, call), [group], dt, xs, cuts, free_and_again=True)
    for i in range(4):
        _close(outs[i], _plain_attention(w, m, xs[i]), rel, f"attention {m} sequence {i}")


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("mask,query,key", [(64, 200, 191), (64, 200, 192), (96, 300, 287), (96, 300, 288), (96, 300, 299),
                                            (0, 500, 0), (0, 500, 63), (0, 500, 64), (0, 130, 127), (50, 149, 99), (50, 149, 100),
                                            (50, 150, 149), (50, 151, 150), (1, 9, 8)])
def test_attention_sees_one_loud_key_inside_its_block_only(dtype, rel, mask, query, key):
    """One key far back, at a block's first or last place, or just outside it, with a score that stands out: queries
    and keys read one half of the input and values the other, and the query's token repeats the loud key's first half.
    Fed whole and with the query decoded alone."""
    from pytorch_transformers_amd.engine.spec import CACHE_FULL, CacheGroupSpec, LayerCall

    m, hidden, dt = attn(2, 1, 24, 20, 0, 1e4, 2.0, mask, False)["mixer"], 32, TORCH[dtype]  # (rotation: the tests above)
    mixer = _attention_mixer(hidden, m)
    w = _part_weights(mixer, seed=6)
    w["a.q"][:, 16:] = 0
    w["a.k"][:, 16:] = 0
    w["a.v"][:, :16] = 0
    w["a.q"][24:] = w["a.q"][:24]
    w["a.k"] = w["a.q"][:24].clone()  # the key of a token points where its heads' queries point
    w["a.g"][:] = 0  # an even gate
    _load_part(mixer, w, dt)
    n = query + 3
    x = _bf16(_rand(n, hidden, seed=7))
    x[:, :16] *= 0.2
    loud = _bf16(_rand(16, seed=8) * 3.0)
    x[key, :16] = loud
    x[query, :16] = loud
    want = _plain_attention(w, m, x)
    quiet = x.clone()
    quiet[key, :16] = x[key - 1 if key else 1, :16]
    visible = mask == 0 or key // mask == query // mask
    moved = float((_plain_attention(w, m, quiet)[query] - want[query]).abs().max()) > 0.3 * float(want[query].abs().max())
    assert moved == (visible and key != query), "the test's loud key does not show where it should"
    group = CacheGroupSpec("kv", CACHE_FULL, 1, 1, mixer.frame)
    call = LayerCall(0, "kv", 0)
    for cuts in ([[n]], [[query, 1, 2]], [[key + 1, query - key - 1, 1, 1, 1]] if query - key > 1 else [[key, 1, 1, 1, 1]]):
        got = _run_in_cuts(lambda t, ctx: mixer.forward(t, ctx, call), [group], dt, [x], cuts)[0]
        _close(got, want, rel, f"block {mask}, query {query}, loud key {key}, cuts {cuts}")


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("shape,cuts", [(lin(), CUTS), (lin(2, 20, 8, (0.8, 0.999)), CUTS), (lin(1, 16, 16, (0.9,)), CUTS),
                                        (lin(3, 70, 72, (0.2, 0.95, 1.0)), CUTS), (lin(), LONG_CUTS)])
def test_linear_attention_mixer_alone(dtype, rel, shape, cuts):
    from pytorch_transformers_amd.engine.spec import CACHE_STATE, CacheGroupSpec, LayerCall
    from pytorch_transformers_amd.parts import DecayLinearAttentionMixer

    m, hidden, dt, eps = shape["mixer"], 32, TORCH[dtype], 1e-5
    mixer = DecayLinearAttentionMixer("a", hidden, m["heads"], m["dim"], m["vdim"], m["decay"], eps)
    w = _part_weights(mixer, seed=9)
    _load_part(mixer, w, dt)
    group = CacheGroupSpec("s", CACHE_STATE, 1, state_shape=mixer.state_shape)
    call = LayerCall(0, "s", 0)
    T = sum(cuts[0])
    xs = [_bf16(_rand(T, hidden, seed=50 + i)) for i in range(len(cuts))]
    outs = _run_in_cuts(lambda x, ctx: mixer.forward(x, ctx, call), [group], dt, xs, cuts, free_and_again=True)
    for i, x in enumerate(xs):
        kept, want = {}, []
        for pos in range(T):
            want.append(P.lightning_token(w, "a", m, eps, x[pos], kept))
        _close(outs[i], torch.stack(want), rel, f"linear attention {m} sequence {i}")


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("rows", [1, 9, 300])
def test_dense_feed_forward_clamps_its_gate(dtype, rel, rows):
    from pytorch_transformers_amd.parts import GatedFeedForward

    hidden, dt = 40, TORCH[dtype]
    for ff, limit in ((56, 0.7), (8, 100.0)):
        part = GatedFeedForward("f", hidden, ff, "clamped", 1.702, limit)
        w = _part_weights(part, seed=11, std=0.4)
        _load_part(part, w, dt)
        x = _bf16(_rand(rows, hidden, seed=12))
        want = torch.stack([P.dense_ff(w, "f", {"limit": limit}, x[i]) for i in range(rows)])
        pre = w["f.gate"] @ x.T
        assert limit > 50 or (float(pre.max()) > limit and float((w["f.up"] @ x.T).min()) < -limit)  # the clamps bite
        _close(part.forward(x.to(dt).cuda(), None), want, rel, f"dense feed-forward ff {ff} limit {limit} rows {rows}")


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("experts,top,scale,ff,hidden", [(5, 2, 1.5, 24, 40), (1, 1, 1.0, 8, 40), (7, 7, 0.5, 16, 40),
                                                         (70, 3, 2.0, 40, 40), (4, 1, 3.0, 9, 40),
                                                         # sizes that the matrix-core launches take (steps of many tokens)
                                                         (5, 2, 1.5, 64, 64), (70, 3, 2.0, 192, 128), (3, 3, 1.0, 320, 64)])
def test_routed_feed_forward(dtype, rel, experts, top, scale, ff, hidden):
    from pytorch_transformers_amd import ops
    from pytorch_transformers_amd.parts import RoutedFeedForward

    dt = TORCH[dtype]
    part = RoutedFeedForward("f", hidden, ff, experts, top, scale)
    w = _part_weights(part, seed=13, std=0.4)
    _load_part(part, w, dt)
    mlp = {"router": {"experts": experts, "top": top, "scale": scale}}
    for rows in (1, 7, 17, 150, 700):
        x = _bf16(_rand(rows, hidden, seed=14 + rows))
        want = torch.stack([P.routed_ff(w, "f", mlp, x[i]) for i in range(rows)])
        _close(part.forward(x.to(dt).cuda(), None), want, rel, f"routed feed-forward {experts} experts top {top} rows {rows}")
        ids, wts = ops.moe_route(x.to(dt).cuda(), part.router, top, "sigmoid", True, scale)
        s = torch.sigmoid(x @ w["f.router"].T)
        best = torch.topk(s, top, dim=1)
        assert torch.equal(ids.cpu().long().sort(dim=1)[0], best.indices.sort(dim=1)[0])
        _close(wts.sum(dim=1), torch.full((rows,), scale, dtype=torch.float64), 1e-5, "the weights add up to the scale")


# ---- whole models ------------------------------------------------------------------------------------------------------
REL_BF16_MODEL = 0.1


def assert_model_close(got, want, rel, what):
    if rel < 1e-3:
        return helpers.assert_close(got, want, rel, what)
    assert got.shape == want.shape and torch.isfinite(got).all(), what
    err, scale = (got.double() - want.double()), float(want.abs().max())
    worst = err.abs().max(dim=1)[0] / scale  # per position
    beyond, middle = int((worst > rel).sum()), float(worst.median())
    # (a sequence of one or two tokens has no median to speak of: a first token's linear attention is a product of two
    # vectors that may all but cancel, and one token in fifty is off by a tenth for that)
    assert beyond <= max(1, got.shape[0] // 10) and (middle <= 0.04 or got.shape[0] < 3), \
        f"{what}: {beyond} of {got.shape[0]} positions beyond {rel} of the largest logit, the median position at {middle:.3f}"


@pytest.mark.parametrize("dtype,rel", [("float32", helpers.REL_F32), ("bfloat16", REL_BF16_MODEL)])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_schedules_give_the_plain_logits(tmp_path, name, dtype, rel):
    """Whole prompts, prompt then token by token, unequal batches decoded together, requests that join and leave
    with prompts in portions down to one token: all the plain logits, with slots and pages freed and used again."""
    from pytorch_transformers_amd.engine.replay import Replayer

    cfg = CONFIGS[name]
    w = make_weights(cfg, seed=11)
    model = load(write_model(tmp_path / name, cfg, w), dtype)
    reqs = helpers.make_requests(cfg["vocab"], [9, 70, 131, 1, 64, 65, 2, 300], seed=3)
    want = plain_all(cfg, w, reqs)
    rp = Replayer(model, 1024, max_slots=8)
    for label, records in (("whole", helpers.schedule_whole(reqs)), ("tail", helpers.schedule_tail(reqs, 40)),
                           ("batches", helpers.schedule_batches(reqs, 3)),
                           ("staggered", helpers.schedule_staggered(reqs, chunks=(None, 2, 19, 1))),
                           ("batches again", helpers.schedule_batches(reqs, 4, decode=(1, 30, 2, 5)))):
        got = helpers.run_schedule(rp, records)
        for rid in reqs:
            assert_model_close(got[rid], want[rid], rel, f"{name} {dtype} {label} {rid}")
        assert not rp.cache.live_slots()


def test_passes_of_a_loop_keep_states_of_their_own(tmp_path):
    """A model whose loop runs its layers three times equals the model that lists those layers three times."""
    cfg = CONFIGS["loop"]
    w = make_weights(cfg, seed=21)
    flat = config(cfg["layers"] * 3, vocab=cfg["vocab"], width=cfg["width"])
    w_flat = {k: v for k, v in w.items() if not k.startswith("l")}
    for rep in range(3):
        for k, v in w.items():
            if k.startswith("l"):
                i, rest = k[1:].split(".", 1)
                w_flat[f"l{int(i) + 3 * rep}.{rest}"] = v
    toks = helpers.make_requests(cfg["vocab"], [90], seed=8)["r0"]
    outs = []
    for name, c, ww in (("loop", cfg, w), ("flat", flat, w_flat)):
        model = load(write_model(tmp_path / name, c, ww), "float32")
        cache = model.new_cache(256)
        slot = cache.alloc()
        outs.append(torch.cat([model.step(cache, [slot], [toks[:50]], "all"), model.step(cache, [slot], [toks[50:]], "all")]))
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_equal_direct_ones(tmp_path, dtype):
    """Decode steps replayed from a captured graph give the bits of the same steps launched one by one, with batches
    that are padded to the captured size (the padding rows move the scratch slot's state, never a sequence's)."""
    from pytorch_transformers_amd.engine.replay import Replayer

    cfg = CONFIGS["mixed"]
    folder = write_model(tmp_path / "m", cfg, make_weights(cfg, seed=12))
    reqs = helpers.make_requests(cfg["vocab"], [9, 30, 70, 3, 41, 12, 25, 8, 19, 33, 50], seed=4)
    records = helpers.schedule_batches(reqs, 3, decode=(5, 2, 8)) + \
        [dict(r, step=r["step"] + 1000) for r in helpers.schedule_batches(reqs, 11, decode=(2, 9, 4))]
    outs = {}
    for graphs in (False, True):
        model = load(folder, dtype)
        assert model.use_graphs
        model.use_graphs = graphs
        rp = Replayer(model, 2048, max_slots=16)
        outs[graphs] = [rp.run(rec) for rec in records]
        torch.cuda.synchronize()
    for rec, a, b in zip(records, outs[False], outs[True]):
        assert (a is None) == (b is None)
        if a is not None:
            assert torch.equal(a, b), f"step {rec['step']}: a captured step differs from the same step launched directly"


@pytest.mark.parametrize("dtype,rel", [("float32", helpers.REL_F32), ("bfloat16", REL_BF16_MODEL)])
def test_long_decoding_and_a_loud_far_token(tmp_path, dtype, rel):
    """300 tokens decoded one by one after a short prompt (states and pages carried over hundreds of steps, many edges
    of the masks' blocks passed), with a token near the start whose embedding is loud."""
    from pytorch_transformers_amd.engine.replay import Replayer

    cfg = CONFIGS["mixed"]
    w = make_weights(cfg, seed=13)
    w["embed"][7] = _bf16(w["embed"][7] * 12.0)
    model = load(write_model(tmp_path / "m", cfg, w), dtype)
    toks = [t if t != 7 else 8 for t in helpers.make_requests(cfg["vocab"], [330], seed=5)["r0"]]
    toks[2] = 7
    reqs = {"long": toks}
    want = plain_all(cfg, w, reqs)
    got = helpers.run_schedule(Replayer(model, 1024, max_slots=2), helpers.schedule_tail(reqs, 300))
    assert_model_close(got["long"], want["long"], rel, f"long decoding {dtype}")


def test_greedy_generation_follows_the_plain_model(tmp_path):
    cfg = CONFIGS["mixed"]
    w = make_weights(cfg, seed=14)
    model = load(write_model(tmp_path / "m", cfg, w), "float32")
    reqs = helpers.make_requests(cfg["vocab"], [5, 17, 2], seed=6)
    out = model.generate(list(reqs.values()), max_new_tokens=12, do_sample=False, eos_token_id=None)
    plain = P.PlainBimepel(cfg, w)
    for seq, toks in zip(out, reqs.values()):
        toks = list(toks)
        state = plain.new_sequence()
        last = [plain.token(state, t) for t in toks][-1]
        for _ in range(12):
            toks.append(int(last.argmax()))
            last = plain.token(state, toks[-1])
        assert list(seq) == toks


def test_random_weights_from_a_configuration_run(tmp_path):
    """The framework's own random-weights mode writes the design's tensor names, and what it writes loads and steps."""
    from safetensors import safe_open

    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.weights import write_random_model

    cfg = AutoConfig.from_dict(CONFIGS["mixed"])
    folder = write_random_model(str(tmp_path / "r"), cfg, seed=1, std=0.1)
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        names = set(f.keys())
    assert {"embed", "final.norm", "l0.shift", "l0.mix.q.norm", "l0.mlp.gate", "l1.mix.norm", "l1.mlp.router", "l1.mlp.e4.up",
            "l2.mlp.e6.down", "l3.mix.g"} <= names
    assert not any(n.startswith(("l3.mlp", "l3.norm2")) or ".experts." in n for n in names)
    for dtype in ("bfloat16", "float32"):
        model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
        cache = model.new_cache(256)
        logits = model.step(cache, [cache.alloc()], [[1, 2, 3]], "all")
        assert logits.shape == (3, cfg.vocab) and torch.isfinite(logits).all()


def test_the_command_line_generates_from_a_model_folder(tmp_path, capsys):
    """``run_generation`` on a folder of this design: greedy tokens as the plain model chooses them."""
    from pytorch_transformers_amd import run_generation

    cfg = CONFIGS["ones"]
    w = make_weights(cfg, seed=15)
    folder = write_model(tmp_path / "m", cfg, w)
    rc = run_generation.main(["--model_name_or_path", folder, "--model_type", "bimepel", "--prompt_ids", "3,1,4,1,5",
                              "--length", "6", "--greedy", "--dtype", "float32"])
    assert rc == 0
    printed = [ln for ln in capsys.readouterr().out.splitlines() if ln and ln[0].isdigit()]
    toks = [3, 1, 4, 1, 5]
    for _ in range(6):
        toks.append(int(P.PlainBimepel(cfg, w).logits(toks)[-1].argmax()))
    assert [int(t) for t in printed[-1].split(",")] == toks


# ---- configurations drawn at random ------------------------------------------------------------------------------------
def draw_config(seed):
    """A small model with sizes that nothing else here hits: widths and feed-forwards that are no multiple of 8, head
    sizes from 8 to 130, head counts and groups that are no power of two, rotations of two elements up to the whole
    head, with and without the ramp, masks of any size, decays up to one, one to nine experts, loops anywhere."""
    import random

    r = random.Random(seed)
    width = r.choice([20, 36, 44, 48, 64, 72, 100])

    def layer():
        if r.random() < 0.55:
            kv = r.choice([1, 2, 3])
            dim = r.choice([8, 12, 16, 24, 40, 64, 72, 130])
            m = {"heads": kv * r.choice([1, 2, 3, 5]), "kv_heads": kv, "dim": dim,
                 "vdim": r.choice([4, 8, 20, 32, 48, 64, 100]), "scale": r.choice([0.1, 0.25, dim ** -0.5])}
            if r.random() < 0.85:
                m["rot"] = {"base": r.choice([100.0, 1e4, 500000.0]), "dims": r.choice([2, dim // 2 // 2 * 2 or 2, dim])}
                if r.random() < 0.6:
                    m["rot"]["scaling"] = {"factor": r.choice([2.0, 8.0]), "original": r.choice([16, 64, 2048]),
                                           "fast": r.choice([32.0, 4.0]), "slow": r.choice([1.0, 0.5])}
            if r.random() < 0.8:
                m["mask"] = {"size": r.choice([1, 3, 16, 33, 64, 65, 128, 1000])}
            out = {"type": "attention", "mixer": m}
        else:
            heads = r.choice([1, 2, 3, 5])
            out = {"type": "lightning", "mixer": {"heads": heads, "dim": r.choice([4, 8, 20, 32, 70]),
                                                  "vdim": r.choice([4, 16, 24, 64, 80]),
                                                  "decay": [r.choice([0.3, 0.9, 0.99, 0.999, 1.0]) for _ in range(heads)]}}
        kind = r.random()
        if kind < 0.15:
            out["mlp"] = None
        elif kind < 0.55:
            out["mlp"] = {"kind": "dense", "ff": r.choice([8, 20, 50, 96]), "limit": r.choice([0.5, 1.0, 7.0])}
        else:
            experts = r.choice([1, 2, 4, 9])
            out["mlp"] = {"kind": "moe", "expert": {"ff": r.choice([4, 12, 32, 64])},
                          "router": {"experts": experts, "top": r.randint(1, experts), "scale": r.choice([0.5, 1.0, 2.5])}}
        return out

    n = r.choice([1, 2, 3, 4])
    cfg = config([layer() for _ in range(n)], vocab=r.choice([61, 97, 211]), width=width, eps=r.choice([1e-5, 1e-6]))
    if r.random() < 0.7:
        a = r.randint(0, n - 1)
        cfg["loop"] = {"start": a, "stop": r.randint(a, n), "times": r.choice([1, 2, 3])}
    return cfg


@pytest.mark.parametrize("seed", range(16))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Whole, cut and batched against the plain model in 32-bit; bfloat16 runs and agrees with itself across schedules
    to rounding (it is held against the plain model where the sizes are the tests' own, above)."""
    from pytorch_transformers_amd.engine.replay import Replayer

    cfg = draw_config(seed)
    w = make_weights(cfg, seed=100 + seed)
    folder = write_model(tmp_path / "m", cfg, w)
    reqs = helpers.make_requests(cfg["vocab"], [5, 70, 140, 1, 66], seed=seed)
    want = plain_all(cfg, w, reqs)
    model = load(folder, "float32")
    rp = Replayer(model, 1024, max_slots=8)
    for label, records in (("whole", helpers.schedule_whole(reqs)), ("batches", helpers.schedule_batches(reqs, 3)),
                           ("staggered", helpers.schedule_staggered(reqs, chunks=(None, 2, 19, 1)))):
        got = helpers.run_schedule(rp, records)
        for rid in reqs:
            helpers.assert_close(got[rid], want[rid], helpers.REL_F32, f"seed {seed} {label} {rid}: {cfg}")
    model = load(folder, "bfloat16")
    rp = Replayer(model, 1024, max_slots=8)
    whole = helpers.run_schedule(rp, helpers.schedule_whole(reqs))
    cut = helpers.run_schedule(rp, helpers.schedule_staggered(reqs, chunks=(None, 2, 19, 1)))
    for rid in reqs:
        assert torch.isfinite(whole[rid]).all()
        assert_model_close(cut[rid], whole[rid], 0.15, f"seed {seed} bfloat16, cut against whole, {rid}: {cfg}")
