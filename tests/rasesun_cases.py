"""Scenarios for the Rasesun family, run by the CPU tests (reference ops,
fp32) and the GPU tests (HIP kernels, fp32 and bf16). Every scenario builds
a small configuration with random weights, runs it through the engine and
compares with the plain model in rasesun_oracle.py."""
import math

import torch

import rasesun_oracle as oracle
from kukeon_amd.engine.config import EngineConfig, SamplingParams
from kukeon_amd.engine.engine import LLMEngine
from kukeon_amd.engine.kv_cache import SequenceKV
from kukeon_amd.models.rasesun import RasesunConfig, RasesunModel


def ssm(heads=4, vdim=8, state=12, groups=2, conv=3, norm_groups=2):
    return {"type": "mamba2",
            "mixer": {"heads": heads, "vdim": vdim, "state": state,
                      "groups": groups, "conv": conv,
                      "norm_groups": norm_groups}}


def latent(heads=3, dim=8, rot_dim=6, rot_dims=None, vdim=10, q_rank=20,
           kv_rank=24, window=7, base=100.0, scale=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim,
                      "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "mask": {"size": window},
                      "rot": {"dims": rot_dims or rot_dim, "base": base},
                      "scale": scale if scale is not None
                      else (dim + rot_dim) ** -0.5}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top}}


def layer(mix, mlp):
    return dict(mix, mlp=mlp)


def config(layers, width=40, vocab=45, scale=2.0, eps=1e-5, loop=None,
           softcap=8.0):
    c = {"architecture": "Rasesun", "width": width, "vocab": vocab,
         "embedding": {"scale": scale}, "norm": {"eps": eps},
         "layers": layers, "logit_softcap": softcap}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


CONFIGS = {
    # both mixers, both feed-forwards, a layer without one, a looped span
    # that holds a recurrent AND an attention layer, a partly rotated key
    "hybrid": lambda: config([
        layer(ssm(), dense(56)),
        layer(latent(rot_dims=4), moe(5, 2, 12)),
        layer(ssm(heads=2, vdim=20, state=40, groups=1, conv=2,
                  norm_groups=1), None),
        layer(latent(heads=2, dim=4, rot_dim=8, vdim=6, q_rank=9,
                     kv_rank=17, window=16, base=30.0), dense(33)),
    ], loop=(1, 3, 3)),
    # state rows spread over 8 lanes, groups == heads, five taps, a latent
    # wider than a workgroup, five heads (a partly filled head group), a
    # window longer than a key chunk, one expert per token, no loop
    "wide": lambda: config([
        layer(ssm(heads=4, vdim=64, state=70, groups=4, conv=5,
                  norm_groups=4), moe(3, 1, 20)),
        layer(latent(heads=5, dim=16, rot_dim=8, vdim=12, q_rank=32,
                     kv_rank=300, window=290), dense(64)),
    ], width=64, vocab=61, scale=1.0, eps=1e-3, softcap=30.0),
    # every width a multiple of 8 or 128: the vector and matrix-core forms
    # of the kernels (16-byte loads, expert tiles), six heads on a head
    # group of four
    "aligned": lambda: config([
        layer(ssm(heads=2, vdim=32, state=16, groups=1, conv=4,
                  norm_groups=2), moe(4, 2, 128)),
        layer(latent(heads=6, dim=16, rot_dim=8, vdim=16, q_rank=24,
                     kv_rank=32, window=20), moe(3, 1, 128)),
    ], width=128, vocab=50, loop=(0, 2, 2)),
    # a latent of 128 with a rotated part of 32: the sizes of the
    # matrix-core attention kernel, which long portions take
    "tiles": lambda: config([
        layer(ssm(heads=2, vdim=16, state=8, groups=2, conv=2,
                  norm_groups=1), None),
        layer(latent(heads=3, dim=8, rot_dim=32, rot_dims=12, vdim=8,
                     q_rank=16, kv_rank=128, window=50), dense(48)),
    ], width=48, vocab=40),
    # no attention at all (no cache pages), and no recurrence at all (no
    # state), a loop that runs once
    "only_ssm": lambda: config([
        layer(ssm(heads=2, vdim=4, state=5, groups=1, conv=3,
                  norm_groups=2), dense(20)),
        layer(ssm(heads=1, vdim=8, state=3, groups=1, conv=2,
                  norm_groups=1), None),
    ], width=16, vocab=21, loop=(0, 1, 1)),
    "only_latent": lambda: config([
        layer(latent(heads=2, dim=4, rot_dim=4, vdim=4, q_rank=6,
                     kv_rank=8, window=6), moe(3, 2, 8)),
        layer(latent(heads=1, dim=8, rot_dim=2, vdim=3, q_rank=5,
                     kv_rank=16, window=300), None),
    ], width=16, vocab=21),
    # the whole stack looped, attention first, window of one, one tap,
    # no embedding scale, no soft cap
    "looped": lambda: _looped(),
}


def _looped():
    c = config([
        layer(latent(heads=1, dim=6, rot_dim=2, vdim=5, q_rank=7, kv_rank=8,
                     window=1), None),
        layer(ssm(heads=3, vdim=5, state=7, groups=3, conv=1,
                  norm_groups=3), moe(4, 3, 9)),
        layer(latent(heads=4, dim=6, rot_dim=4, vdim=8, q_rank=10,
                     kv_rank=12, window=5), moe(2, 2, 16)),
    ], width=30, vocab=33, loop=(0, 3, 2))
    del c["embedding"]
    del c["logit_softcap"]
    return c


def weights(cfg, seed=0):
    """Random checkpoint for a config dictionary, bf16 like a stored one."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    V = cfg["vocab"]

    def r(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(
            torch.bfloat16)

    t = {"embed": r(V, W), "final.norm": r(W, std=0.2, mean=1.0),
         "head": r(V, W, std=2.0 * W ** -0.5)}
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = L["mixer"]
        t[p + "norm1"] = r(W, std=0.2, mean=1.0)
        t[p + "norm1b"] = r(W, std=0.2, mean=0.7)
        q = p + "mix."
        if L["type"] == "mamba2":
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, C = H * P, H * P + 2 * G * N
            t[q + "in"] = r(2 * inner + 2 * G * N + H, W, std=1.5 * W ** -0.5)
            t[q + "conv"] = r(C, m["conv"], std=0.6)
            t[q + "conv.b"] = r(C, std=0.3)
            t[q + "dt_bias"] = r(H, std=0.8, mean=-1.0)
            t[q + "A_log"] = r(H, std=0.7, mean=-0.5)
            t[q + "D"] = r(H, std=0.5, mean=1.0)
            t[q + "norm"] = r(inner, std=0.2, mean=1.0)
            t[q + "o"] = r(W, inner, std=inner ** -0.5)
        else:
            H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            Rq, R = m["q_rank"], m["kv_rank"]
            t[q + "dq"] = r(Rq, W, std=W ** -0.5)
            t[q + "dq.norm"] = r(Rq, std=0.2, mean=1.0)
            t[q + "uq"] = r(H * (dn + dr), Rq, std=2.0 * Rq ** -0.5)
            t[q + "dkv"] = r(R + dr, W, std=W ** -0.5)
            t[q + "dkv.norm"] = r(R, std=0.2, mean=1.0)
            t[q + "uk"] = r(H * dn, R, std=2.0 * R ** -0.5)
            t[q + "uv"] = r(H * dv, R, std=R ** -0.5)
            t[q + "g"] = r(H, W, std=W ** -0.5)
            t[q + "o"] = r(W, H * dv, std=(H * dv) ** -0.5)
        f = L["mlp"]
        if not f:
            continue
        t[p + "norm2"] = r(W, std=0.2, mean=1.0)
        t[p + "norm2b"] = r(W, std=0.2, mean=0.7)
        q = p + "mlp."
        if f["kind"] == "dense":
            t[q + "up"] = r(f["ff"], W, std=1.5 * W ** -0.5)
            t[q + "down"] = r(W, f["ff"], std=f["ff"] ** -0.5)
            t[q + "act"] = r(2, std=0.7)
        else:
            E, top, ff = f["router"]["experts"], f["router"]["top"], \
                f["expert"]["ff"]
            for e in range(E):
                t[q + f"e{e}.up"] = r(ff, W, std=1.5 * W ** -0.5)
                t[q + f"e{e}.down"] = r(W, ff, std=ff ** -0.5)
            t[q + "table"] = torch.stack(
                [torch.randperm(E, generator=g)[:top] for _ in range(V)]
            ).to(torch.int32)
    return t


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def _poison(eng):
    # whatever a sequence has not written itself must never be read
    for t in eng.kv.k:
        if t is not None:
            t.fill_(300.0)
    for st in eng.states.layers:
        if st is not None:
            for t in (st if isinstance(st, tuple) else (st,)):
                t.fill_(-700.0)


def make_engine(cfg, tensors, device, dtype, blocks=96, slots=4,
                block_size=4, max_len=384, poison=True, **ekw):
    mcfg = RasesunConfig.from_json(cfg)
    model = RasesunModel(mcfg, device=device, dtype=dtype, tensors=tensors,
                         max_position=max_len)
    kw = dict(block_size=block_size, max_model_len=max_len,
              max_sessions=slots, state_slots=slots, num_kv_blocks=blocks,
              use_graphs=False)
    kw.update(ekw)
    eng = LLMEngine(model, mcfg, EngineConfig(**kw), device=device)
    if poison:
        _poison(eng)
    return eng


def tol(dtype):
    return 2e-4 if dtype == "fp32" else 0.12


def rel_err(got, want):
    """Error of logits rows as the ratio of centred root mean squares."""
    got = got.detach().cpu().double()
    want = want.detach().cpu().double()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() /
                  w.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())


def check(got, want, dtype, what=""):
    e = rel_err(got, want)
    assert e <= tol(dtype), f"{what}: error {e:.3g} over {tol(dtype)}"


def run_schedule(eng, prompts, schedule):
    """schedule: list of steps, each a list of (request index, count).
    -> per request the logits at every position [len, vocab]. A request is
    freed when it is through."""
    bs = eng.ecfg.block_size
    kvs, at = {}, {}
    out = {i: [] for i in range(len(prompts))}
    for step in schedule:
        entries, want = [], []
        for i, n in step:
            if i not in kvs:
                kvs[i] = SequenceKV(bs)
                at[i] = 0
            entries.append((kvs[i], prompts[i][at[i]: at[i] + n]))
            want.append(list(range(n)))
        lg = eng.forward_tokens(entries, want)
        row = 0
        for i, n in step:
            out[i].append(lg[row: row + n])
            row += n
            at[i] += n
            if at[i] == len(prompts[i]):
                eng.free_sequence(kvs.pop(i))
    return {i: torch.cat(v) for i, v in out.items() if v}


def portions(total, sizes):
    out, k = [], 0
    while total > 0:
        n = min(sizes[k % len(sizes)], total)
        out.append(n)
        total -= n
        k += 1
    return out


# ---------------------------------------------------------------- scenarios
def case_whole(name, device, dtype, n=27):
    cfg = CONFIGS[name]()
    W = weights(cfg, 1)
    toks = tokens(cfg, n, 1)
    eng = make_engine(cfg, W, device, dtype)
    got = run_schedule(eng, [toks], [[(0, len(toks))]])[0]
    check(got, oracle.forward(cfg, W, toks), dtype, name)


def case_layers(device, dtype):
    """The residual stream after every layer run."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 2)
    toks = tokens(cfg, 11, 2)
    eng = make_engine(cfg, W, device, dtype)
    want = []
    oracle.forward(cfg, W, toks, taps=want)
    assert len(want) == 1 + 2 * 3 + 1
    kv = SequenceKV(eng.ecfg.block_size)
    got = []
    fwd = eng.model.forward
    eng.model.forward = lambda *a, **k: fwd(*a, taps=got, **k)
    eng.forward_tokens([(kv, toks)])
    eng.model.forward = fwd
    assert len(got) == len(want)
    for i, (g, w) in enumerate(zip(got, want)):
        e = float((g.cpu().double() - w).abs().max() / w.abs().max())
        assert e <= tol(dtype), f"layer run {i}: {e:.3g}"


def case_prefill_vs_decode(name, device, dtype):
    cfg = CONFIGS[name]()
    W = weights(cfg, 3)
    toks = tokens(cfg, 25, 3)
    want = oracle.forward(cfg, W, toks)
    whole = run_schedule(make_engine(cfg, W, device, dtype), [toks],
                         [[(0, len(toks))]])[0]
    one = run_schedule(make_engine(cfg, W, device, dtype), [toks],
                       [[(0, 1)] for _ in toks])[0]
    check(whole, want, dtype, "whole")
    check(one, want, dtype, "token by token")
    check(one, whole, dtype, "token by token against whole")


def case_portions(name, device, dtype, sizes, n=41):
    cfg = CONFIGS[name]()
    W = weights(cfg, 4)
    toks = tokens(cfg, n, 4)
    sched = [[(0, k)] for k in portions(len(toks), sizes)]
    got = run_schedule(make_engine(cfg, W, device, dtype), [toks], sched)[0]
    check(got, oracle.forward(cfg, W, toks), dtype, f"portions {sizes}")


def case_batch(name, device, dtype):
    """Unequal requests in one batch, portions beside single tokens."""
    cfg = CONFIGS[name]()
    W = weights(cfg, 5)
    prompts = [tokens(cfg, n, 10 + n) for n in (19, 1, 7, 30)]
    sched = [
        [(0, 5), (1, 1), (3, 2)],
        [(0, 1), (2, 7), (3, 9)],
        [(3, 1), (0, 1)],
        [(0, 12), (3, 1)],
        [(3, 17)],
    ]
    got = run_schedule(make_engine(cfg, W, device, dtype), prompts, sched)
    for i, p in enumerate(prompts):
        check(got[i], oracle.forward(cfg, W, p), dtype, f"request {i}")


def case_reuse(device, dtype):
    """A pool too small for all requests at once: pages and state slots of
    finished requests are handed to the next ones."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 6)
    prompts = [tokens(cfg, n, 20 + n) for n in (14, 11, 16, 3, 13)]
    eng = make_engine(cfg, W, device, dtype, blocks=8, slots=2, block_size=4)
    sched = [
        [(0, 6), (1, 4)],
        [(0, 8), (1, 1)],          # 0 ends: 4 pages and a slot come back
        [(1, 6), (2, 9)],          # 1 ends
        [(2, 7), (3, 2)],          # 2 ends
        [(3, 1), (4, 12)],         # 3 ends
        [(4, 1)],
    ]
    got = run_schedule(eng, prompts, sched)
    for i, p in enumerate(prompts):
        check(got[i], oracle.forward(cfg, W, p), dtype, f"request {i}")
    assert eng.kv.allocator.num_free == 8 and eng.states.num_free == 2


def case_first_tokens(device, dtype):
    """Sequences shorter than the convolution and the window, started in
    used slots, and a start cut into single tokens."""
    cfg = CONFIGS["wide"]()         # 5 taps
    W = weights(cfg, 7)
    eng = make_engine(cfg, W, device, dtype, slots=1)
    for n, sched in ((1, [1]), (2, [2]), (3, [1, 2]), (9, [1, 1, 1, 2, 4]),
                     (6, [2, 1, 3])):
        toks = tokens(cfg, n, 30 + n)
        got = run_schedule(eng, [toks], [[(0, k)] for k in sched])[0]
        check(got, oracle.forward(cfg, W, toks), dtype, f"length {n}")


def case_long_decode(device, dtype):
    """Decoding far past the windows and through many pages."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 8)
    toks = tokens(cfg, 75, 8)
    sched = [[(0, 3)]] + [[(0, 1)] for _ in range(72)]
    got = run_schedule(make_engine(cfg, W, device, dtype, block_size=4),
                       [toks], sched)[0]
    check(got, oracle.forward(cfg, W, toks), dtype, "long decode")


def case_window_chunks(device, dtype):
    """A window longer than one pass of the attention kernel over the keys,
    prompts longer than the window, portions that end inside it."""
    cfg = CONFIGS["wide"]()
    W = weights(cfg, 9)
    toks = tokens(cfg, 330, 9)
    want = oracle.forward(cfg, W, toks)
    eng = make_engine(cfg, W, device, dtype, blocks=200, max_len=400)
    got = run_schedule(eng, [toks], [[(0, 330)]])[0]
    check(got, want, dtype, "whole")
    sched = [[(0, 255)], [(0, 2)], [(0, 40)]] + [[(0, 1)]] * 33
    got = run_schedule(eng, [toks], sched)[0]
    check(got, want, dtype, "portions and decoding")


def case_grouped_experts(device, dtype):
    """Long portions sort their rows by expert and run each expert over its
    rows at once; short ones go token by token. Both against the plain
    model, two experts per token, two requests in the long step."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 12)
    prompts = [tokens(cfg, n, 70 + n) for n in (90, 71)]
    want = [oracle.forward(cfg, W, p) for p in prompts]
    eng = make_engine(cfg, W, device, dtype, blocks=64, max_len=128)
    got = run_schedule(eng, prompts, [[(0, 90), (1, 70)], [(1, 1)]])
    for i in range(2):
        check(got[i], want[i], dtype, f"sorted rows, request {i}")
    a, b = portions(90, (7,)), portions(71, (5, 1))
    sched = [[(i, c[k]) for i, c in ((0, a), (1, b)) if k < len(c)]
             for k in range(max(len(a), len(b)))]
    got = run_schedule(eng, prompts, sched)
    for i in range(2):
        check(got[i], want[i], dtype, f"token by token, request {i}")


def case_long_portions(device, dtype):
    """Portions long enough for the matrix-core attention kernel beside
    short ones and single tokens that take the other forms."""
    cfg = CONFIGS["tiles"]()
    W = weights(cfg, 13)
    prompts = [tokens(cfg, n, 80 + n) for n in (560, 70)]
    want = [oracle.forward(cfg, W, p) for p in prompts]
    eng = make_engine(cfg, W, device, dtype, blocks=48, block_size=16,
                      max_len=640)
    got = run_schedule(eng, prompts, [[(0, 560), (1, 69)], [(1, 1)]])
    for i in range(2):
        check(got[i], want[i], dtype, f"whole, request {i}")
    got = run_schedule(eng, prompts,
                       [[(0, 21)], [(0, 530), (1, 2)], [(0, 1), (1, 68)],
                        [(0, 8)]])
    for i in range(2):
        check(got[i], want[i], dtype, f"portions, request {i}")


def case_greedy(device, dtype, graphs=False):
    """Generation through add_request / step with the greedy sampler."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 10)
    eng = make_engine(cfg, W, device, dtype, blocks=64, max_len=128,
                      poison=False, use_graphs=graphs, graph_buckets=(4,),
                      decode_microbatch=4, max_prefill_tokens=16)
    prompts = [tokens(cfg, n, 40 + n) for n in (5, 21, 2)]
    sp = SamplingParams(temperature=0.0, max_new_tokens=8)
    rids = {}
    for i, p in enumerate(prompts):
        rids[eng.add_request(SequenceKV(4), p, sp)] = i
    out = {i: [] for i in range(len(prompts))}
    while eng.has_work():
        for o in eng.step():
            out[rids[o.req_id]].extend(o.new_tokens)
    for i, p in enumerate(prompts):
        want = oracle.greedy(cfg, W, p, 8)
        if dtype == "fp32":
            assert out[i] == want, f"request {i}: {out[i]} != {want}"
        else:
            # bf16 may flip a near-tie; the first tokens still agree
            assert out[i][:2] == want[:2], f"request {i}"


def assert_greedy(cfg, W, prompt, got, what=""):
    """Every generated token is the plain model's best one, up to the
    rounding of the logits to bfloat16 that the sampler works on."""
    toks = list(prompt)
    for i, t in enumerate(got):
        lg = oracle.forward(cfg, W, toks)[-1]
        best = float(lg.max())
        assert float(lg[t]) >= best - abs(best) * 2.0 ** -7, \
            f"{what}: token {i} is {t}, the plain model says " \
            f"{int(lg.argmax())}"
        toks.append(t)


def _generate(eng, kv, prompt, n):
    sp = SamplingParams(temperature=0.0, max_new_tokens=n)
    eng.add_request(kv, prompt, sp)
    out = []
    while eng.has_work():
        for o in eng.step():
            out.extend(o.new_tokens)
    return out


def case_multi_turn(device, dtype):
    """A session's second turn continues from its pages and state slots; an
    idle session whose pages and slot were taken away is rebuilt from its
    history."""
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 15)
    eng = make_engine(cfg, W, device, dtype, blocks=12, slots=2, max_len=64,
                      poison=False, decode_microbatch=2)
    a, b = SequenceKV(4), SequenceKV(4)
    p1, p2, p3 = tokens(cfg, 9, 60), tokens(cfg, 5, 61), tokens(cfg, 30, 62)
    t1 = _generate(eng, a, p1, 4)
    assert_greedy(cfg, W, p1, t1, "first turn")
    t2 = _generate(eng, a, p2, 3)
    assert_greedy(cfg, W, p1 + t1 + p2, t2, "second turn")
    assert a.num_tokens > 0 and a.state_slot >= 0
    # b needs more pages than are left: a's pages and slot are taken
    tb = _generate(eng, b, p3, 4)
    assert_greedy(cfg, W, p3, tb, "other session")
    assert a.num_tokens == 0 and a.state_slot < 0 and a.history
    eng.free_sequence(b)
    t3 = _generate(eng, a, [7, 3], 3)
    assert len(t1) == 4 and len(t2) == 3 and len(tb) == 4 and len(t3) == 3
    assert_greedy(cfg, W, p1 + t1 + p2 + t2 + [7, 3], t3, "rebuilt session")


def case_modelhub(device):
    """The serving daemon's model server with this family: sessions over the
    unix socket, two turns on one session, greedy tokens as the plain model
    gives them."""
    import uuid
    from kukeon_amd.serve.server import ModelhubClient, ModelhubServer
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 16)
    mcfg = RasesunConfig.from_json(cfg)
    model = RasesunModel(mcfg, device=device, dtype="fp32", tensors=W,
                         max_position=128)
    ecfg = EngineConfig(block_size=4, max_model_len=128, max_sessions=4,
                        state_slots=4, num_kv_blocks=64, use_graphs=False)
    sock = f"/tmp/mh-{uuid.uuid4().hex[:10]}.sock"
    hub = ModelhubServer(model, mcfg, ecfg, sock, device=device)
    hub.start()
    try:
        c = ModelhubClient(sock, timeout=120)
        p1, p2 = tokens(cfg, 6, 70), tokens(cfg, 3, 71)
        r1 = c.generate("s", p1, max_new_tokens=4, temperature=0.0)
        assert len(r1["tokens"]) == 4
        assert_greedy(cfg, W, p1, r1["tokens"], "first turn")
        r2 = c.generate("s", p2, max_new_tokens=3, temperature=0.0)
        assert len(r2["tokens"]) == 3
        assert_greedy(cfg, W, p1 + r1["tokens"] + p2, r2["tokens"],
                      "second turn")
        rb = c.generate("t", p2, max_new_tokens=2, temperature=0.0)
        assert len(rb["tokens"]) == 2
        assert_greedy(cfg, W, p2, rb["tokens"], "other session")
        assert c.call("stats")["sessions"] == 2
        c.close()
    finally:
        hub.stop()


def write_checkpoint(folder, cfg, W):
    """config.json and model.safetensors (8-byte header length, JSON header,
    raw data) of a config dictionary and its tensors."""
    import json
    import os
    import struct
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    head, blobs, at = {}, [], 0
    for name, t in W.items():
        raw = (t.view(torch.int16) if t.dtype == torch.bfloat16 else t) \
            .contiguous().numpy().tobytes()
        head[name] = {"dtype": "BF16" if t.dtype == torch.bfloat16
                      else "I32", "shape": list(t.shape),
                      "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(head).encode()
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))


def case_trace_runner(tmp_path, device, dtype):
    """The trace runner as a program: a checkpoint folder, steps on standard
    input, logits files and `done` lines back. Three requests through a pool
    sized for two, portions beside single tokens, a request left out of a
    step."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    cfg = CONFIGS["hybrid"]()
    W = weights(cfg, 14)
    model_dir = tmp_path / "model"
    out_dir = tmp_path / "out"
    model_dir.mkdir()
    write_checkpoint(model_dir, cfg, W)
    prompts = {"a": tokens(cfg, 70, 90), "b": tokens(cfg, 40, 91),
               "c": tokens(cfg, 33, 92)}
    want = {k: oracle.forward(cfg, W, p) for k, p in prompts.items()}
    steps = [[("a", 30), ("b", 1)], [("a", 1), ("b", 38)], [("a", 39)],
             [("b", 1), ("c", 2)], [("c", 30)], [("c", 1)]]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cmd = [sys.executable, os.path.join(root, "bin", "trace_run"), "--model",
           str(model_dir), "--dtype",
           "float32" if dtype == "fp32" else "bfloat16", "--out",
           str(out_dir), "--max-tokens", "128", "--slots", "2", "--device",
           device]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                         text=True, cwd=root)
    at = {k: 0 for k in prompts}
    try:
        for n, step in enumerate(steps):
            entries, end = [], []
            for k, cnt in step:
                toks = prompts[k][at[k]: at[k] + cnt]
                entries.append({"id": k, "tokens": toks,
                                "want": [0, cnt - 1] if cnt > 1 else [0]})
                at[k] += cnt
                if at[k] == len(prompts[k]):
                    end.append(k)
            p.stdin.write(json.dumps({"step": n, "entries": entries,
                                      "end": end}) + "\n")
            p.stdin.flush()
            line = p.stdout.readline()
            while line and line.strip() != "done %d" % n:
                line = p.stdout.readline()
            assert line, "the runner ended early"
            got = np.fromfile(out_dir / ("%d.f32" % n), dtype="<f4").reshape(
                -1, cfg["vocab"])
            row = 0
            for k, cnt in step:
                a = at[k] - cnt
                for w in ([0, cnt - 1] if cnt > 1 else [0]):
                    check(torch.from_numpy(got[row].copy())[None],
                          want[k][a + w][None], dtype, f"step {n} {k}+{w}")
                    row += 1
            assert row == got.shape[0]
        p.stdin.close()
        assert p.wait(timeout=60) == 0
    finally:
        if p.poll() is None:
            p.kill()


def case_registry(tmp_path, device, dtype):
    """A checkpoint folder is found by its architecture name and read."""
    from kukeon_amd.models.registry import load_checkpoint
    cfg = CONFIGS["looped"]()
    W = weights(cfg, 11)
    write_checkpoint(tmp_path, cfg, W)
    mcfg, model = load_checkpoint(str(tmp_path), device=device, dtype=dtype)
    assert mcfg.family == "rasesun" and len(model.runs) == 6
    eng = LLMEngine(model, mcfg, EngineConfig(
        block_size=4, max_model_len=64, max_sessions=2, state_slots=2,
        num_kv_blocks=16, use_graphs=False), device=device)
    toks = tokens(cfg, 13, 11)
    got = run_schedule(eng, [toks], [[(0, 6)], [(0, 7)]])[0]
    check(got, oracle.forward(cfg, W, toks), dtype, "from a folder")


# ------------------------------------------------------- single mechanisms
def _act(dtype):
    return torch.float32 if dtype == "fp32" else torch.bfloat16


def _close(got, want, dtype, what, scale=None):
    got = got.detach().cpu().double()
    want = want.detach().cpu().double()
    ref = float(want.abs().max()) if scale is None else scale
    e = float((got - want).abs().max()) / max(ref, 1e-9)
    lim = 2e-5 if dtype == "fp32" else 2e-2
    assert e <= lim, f"{what}: error {e:.3g} over {lim}"


def _i32(x, device):
    return torch.tensor(x, dtype=torch.int32, device=device)


def case_op_sandwich_norm(device, dtype):
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(0)
    for rows, W in ((5, 33), (1, 1), (3, 600), (2, 2056)):
        x = torch.randn(rows, W, generator=g) * 3
        y = (torch.randn(rows, W + 3, generator=g) * 5).to(_act(dtype))
        pw = torch.randn(W, generator=g)
        w = torch.randn(W, generator=g)
        xd = x.clone().to(device)
        out = torch.empty(rows, W, dtype=_act(dtype), device=device)
        ops.postnorm_residual_rmsnorm(xd, y.to(device)[:, :W], pw.to(device),
                                      w.to(device), 1e-3, out)
        s = x.double() + oracle.rms_norm(y[:, :W].double(), pw, 1e-3)
        _close(xd, s, "fp32", "residual sum")
        _close(out, oracle.rms_norm(s, w, 1e-3), dtype, "norm")
        o2 = torch.empty(rows, W, dtype=_act(dtype), device=device)
        x2 = x.clone().to(device)
        ops.norm_only(x2, w.to(device), 1e-3, o2)
        assert torch.equal(x2.cpu(), x)
        _close(o2, oracle.rms_norm(x.double(), w, 1e-3), dtype, "norm alone")


def case_op_conv(device, dtype, taps=4, cuts=((5, 1, 2, 1, 6), (3, 1, 9, 1)),
                 C=37, col0=5, ld=50):
    """Two sequences cut into portions; the portions of a step share one
    launch; slots start out dirty."""
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(taps)
    act = _act(dtype)
    lens = [sum(c) for c in cuts]
    full = [torch.randn(n, ld, generator=g).to(act) for n in lens]
    cw = torch.randn(C, taps, generator=g) * 0.7
    bias = torch.randn(C, generator=g)
    state = torch.full((3, taps - 1, C), -55.0, device=device)
    zero = torch.zeros(C, device=device)
    slots = [2, 0]
    at = [0, 0]
    got = [[], []]
    for st in range(max(len(c) for c in cuts)):
        seqs = [s for s in range(2) if st < len(cuts[s])]
        rows, pos, rseq, cu = [], [], [], [0]
        for k, s in enumerate(seqs):
            n = cuts[s][st]
            rows.append(full[s][at[s]: at[s] + n])
            pos += list(range(at[s], at[s] + n))
            rseq += [k] * n
            cu.append(cu[-1] + n)
        proj = torch.cat(rows).to(device)
        out = torch.empty(proj.shape[0], C, dtype=act, device=device)
        a = (_i32(pos, device), _i32(rseq, device), _i32(cu, device),
             _i32([slots[s] for s in seqs], device))
        one = all(cuts[s][st] == 1 for s in seqs)   # one launch does both
        ops.conv_act(out, proj, col0, cw.t().contiguous().to(device),
                     bias.to(device), state, *a, 1, one)
        if not one:
            ops.conv_tail_update(state, proj, col0, zero, a[0], a[2], a[3])
        for k, s in enumerate(seqs):
            got[s].append(out[cu[k]: cu[k + 1]].cpu())
            at[s] += cuts[s][st]
    for s in range(2):
        u = full[s][:, col0: col0 + C].double()
        want = oracle.silu(oracle.causal_conv(u, cw, bias))
        _close(torch.cat(got[s]), want, dtype, f"sequence {s}")
    if taps > 1:
        assert float((state[1] + 55.0).abs().max()) == 0.0  # nobody's slot


def case_op_scan(device, dtype, H=3, P=5, N=7, G=3, cuts=(4, 1, 9, 1, 1)):
    """The scan over portions against the scan over the whole sequence; a
    second sequence rides along; the slot starts out dirty; an inactive row
    changes nothing."""
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(H * 100 + N)
    act = _act(dtype)
    T = sum(cuts)
    inner = H * P
    xbc = torch.randn(T, inner + 2 * G * N, generator=g).to(act)
    dt = (torch.randn(T, H + 3, generator=g) * 1.5).to(act)
    dt_bias = torch.randn(H, generator=g)
    a_log = torch.randn(H, generator=g) * 0.5
    skip = torch.randn(H, generator=g)
    xd, B, C = (xbc[:, :inner].double().view(T, H, P),
                xbc[:, inner: inner + G * N].double().view(T, G, N),
                xbc[:, inner + G * N:].double().view(T, G, N))
    per = H // G
    want, S = oracle.selective_scan(
        xd, B.repeat_interleave(per, 1), C.repeat_interleave(per, 1),
        dt[:, 1: 1 + H].double(), dt_bias.double(), a_log.double(),
        skip.double())
    state = torch.full((3, H, P, N), 9.0, device=device)
    got, at = [], 0
    other = torch.randn(1, inner + 2 * G * N, generator=g).to(act)
    for k, n in enumerate(cuts):
        rows = torch.cat([other, xbc[at: at + n]]).to(device)
        dts = torch.cat([dt[:1], dt[at: at + n]]).to(device)
        y = torch.full((n + 1, inner), 5.0, device=device)
        # the first sequence is inactive in odd steps, a fresh one otherwise
        pos = [(-1 if k % 2 else 0)] + list(range(at, at + n))
        before = state[0].clone()
        ops.ssm_scan(y, rows, dts[:, 1: 1 + H], dt_bias.to(device),
                     torch.exp(a_log).to(device), skip.to(device), state,
                     _i32(pos, device), _i32([0, 1, n + 1], device),
                     _i32([0, 2], device), H, P, N, G)
        if k % 2:
            assert torch.equal(state[0], before)
            assert float((y[0] - 5.0).abs().max()) == 0.0
        got.append(y[1:].cpu())
        at += n
    _close(torch.cat(got), want.reshape(T, inner), dtype, "scan outputs")
    _close(state[2].transpose(1, 2), S, dtype, "final state")
    assert float((state[1] - 9.0).abs().max()) == 0.0


def case_op_gated_norm(device, dtype):
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(3)
    for rows, C, parts in ((4, 24, 3), (2, 7, 1), (3, 600, 2), (1, 5, 5),
                           (3, 4800, 2), (2, 5000, 1)):
        y = torch.randn(rows, C, generator=g) * 2
        off = 8 if C % 8 == 0 else 2       # aligned rows take vector loads
        z = torch.randn(rows, C + 2 * off, generator=g).to(_act(dtype))
        w = torch.randn(C, generator=g)
        out = torch.empty(rows, C, dtype=_act(dtype), device=device)
        ops.gated_group_rmsnorm(out, y.to(device),
                                z.to(device)[:, off: off + C], w.to(device),
                                parts, 1e-4)
        v = y.double() * oracle.silu(z[:, off: off + C].double())
        want = oracle.rms_unit(v.view(rows, parts, C // parts), 1e-4).view(
            rows, C) * w.double()
        _close(out, want, dtype, f"gated norm {C}/{parts}")


def case_op_activations(device, dtype):
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(4)
    p, q = 0.3, -0.8
    ap = math.log1p(math.exp(p))
    aq = 0.5 + math.log1p(math.exp(q))
    for width in (52, 51):          # whole 16-byte chunks, and not
        z = (torch.randn(6, width, generator=g) * 3).to(_act(dtype))
        z[0, :4] = torch.tensor([0.0, -0.0, 1e-3, -1e-3]).to(_act(dtype))
        out = torch.empty_like(z, device=device)
        ops.xielu(out, z.to(device), ap, aq)
        _close(out, oracle.xielu(z.double(), p, q), dtype, "xielu")
    lg = torch.randn(3, 40, generator=g) * 40
    ld = lg.clone().to(device)
    ops.softcap_(ld, 25.0)
    _close(ld, 25.0 * torch.tanh(lg.double() / 25.0), "fp32", "soft cap")
    for dv in (6, 16):
        o = torch.randn(3, 5, dv, generator=g).to(_act(dtype))
        gate = torch.randn(5, 3 + 2, generator=g).to(_act(dtype))
        out = torch.empty(5, 3 * dv, dtype=_act(dtype), device=device)
        ops.head_gate(out, o.to(device), gate.to(device)[:, 1:4])
        want = (o.double().permute(1, 0, 2) *
                torch.sigmoid(gate[:, 1:4].double())[:, :, None]).reshape(
                    5, 3 * dv)
        _close(out, want, dtype, "head gate")
    # rows gathered, squared and folded back (the sorted form of the experts)
    for W in (24, 21):
        src = torch.randn(7, W, generator=g).to(_act(dtype))
        rmap = torch.tensor([3, 3, 0, 6, 1, 2], dtype=torch.int32)
        got = torch.empty(6, W, dtype=_act(dtype), device=device)
        ops.gather_rows(got, src.to(device), rmap.to(device))
        assert torch.equal(got.cpu(), src[rmap.long()])
        ops.relu_square_(got)
        _close(got, torch.relu(src[rmap.long()].double()) ** 2, dtype,
               "relu squared")
        inv = torch.tensor([[5, 0], [2, 2], [4, 1]], dtype=torch.int32)
        out = torch.empty(3, W, dtype=_act(dtype), device=device)
        ops.combine_rows(out, got, inv.to(device))
        _close(out, got.cpu().double()[inv.long()].mean(1), dtype,
               "rows folded")


def case_op_table_moe(device, dtype, E=5, top=2, W=24, ff=13, V=11, rows=9):
    from kukeon_amd import ops
    g = torch.Generator().manual_seed(E * 10 + top)
    act = _act(dtype)
    t = {f"e{e}.up": (torch.randn(ff, W, generator=g) * W ** -0.5).to(act)
         for e in range(E)}
    t.update({f"e{e}.down": (torch.randn(W, ff, generator=g)).to(act)
              for e in range(E)})
    t["table"] = torch.stack([torch.randperm(E, generator=g)[:top]
                              for _ in range(V)]).to(torch.int32)
    ids = torch.randint(0, V, (rows,), generator=g)
    h = torch.randn(rows, W, generator=g).to(act)
    out = torch.empty(rows, W, dtype=act, device=device)
    ops.table_moe(out, h.to(device), ids.to(torch.int32).to(device),
                  t["table"].to(device),
                  torch.stack([t[f"e{e}.up"] for e in range(E)]).to(device),
                  torch.stack([t[f"e{e}.down"] for e in range(E)]).to(device))
    f = {"router": {"experts": E, "top": top}}
    want = oracle.table_moe(h.double(), ids.tolist(), f, t, "")
    _close(out, want, dtype, f"table moe top {top}")


def case_op_latent_append(device, dtype):
    from kukeon_amd import ops
    from kukeon_amd.models.rotary import angle_table
    g = torch.Generator().manual_seed(5)
    act = _act(dtype)
    Rq, R, dr, dims, BS, nb = 9, 13, 8, 6, 4, 10
    n = 11
    proj = torch.randn(n, 3 + Rq + 2 + R + dr + 1, generator=g).to(act)
    qc, kc = 3, 3 + Rq + 2
    wq = torch.randn(Rq, generator=g)
    wkv = torch.randn(R, generator=g)
    cs = angle_table(64, dims, 50.0).to(device)
    cache = torch.full((nb, 1, BS, R + dr), 77.0, dtype=act, device=device)
    perm = torch.randperm(nb, generator=g).tolist()
    bt = _i32([perm[:5], perm[5:]], device)
    pos = list(range(20, 20 + n))          # starts at the first slot of a page
    pos[4] = -1                            # an inactive row
    seq = [1] * n
    cq = torch.full((n, Rq), 3.0, dtype=act, device=device)
    ops.latent_kv_append(cq, cache, proj.to(device), qc, kc, wq.to(device),
                         wkv.to(device), 1e-4, cs, _i32([p if p < 0 else p - 20 + 3 for p in pos], device),
                         _i32(seq, device), bt)
    pd = proj.double()
    live = [i for i in range(n) if pos[i] >= 0]
    p_eff = torch.tensor([pos[i] - 20 + 3 for i in live])
    _close(cq[live], oracle.rms_norm(pd[live, qc: qc + Rq], wq, 1e-4), dtype,
           "query latent")
    assert float((cq[4].float() - 3.0).abs().max()) == 0.0
    cw = oracle.rms_norm(pd[live, kc: kc + R], wkv, 1e-4)
    kr = oracle.rotate_pairs(pd[live, kc + R: kc + R + dr], p_eff, dims, 50.0)
    rows = torch.stack([cache[perm[5 + int(p) // BS], 0, int(p) % BS]
                        for p in p_eff])
    _close(rows[:, :R], cw, dtype, "latent")
    _close(rows[:, R:], kr, dtype, "rotated key part")
    untouched = set(range(nb)) - {perm[5 + int(p) // BS] for p in p_eff}
    for b in untouched:
        assert float((cache[b].float() - 77.0).abs().max()) == 0.0


def case_op_latent_attention(device, dtype, ctx=300, BS=16, H=5, R=24, dr=6,
                             window=40):
    """One key is made to dominate a head's scores: far back but inside the
    window, at page borders, the oldest key inside the window and the first
    one outside it (which must stay unseen). Rows are checked as a prompt's
    rows and as single decoded rows."""
    from kukeon_amd import ops
    from kukeon_amd.models.rotary import angle_table
    g = torch.Generator().manual_seed(ctx + window)
    act = _act(dtype)
    dn, dims, base = 3, 4, 20.0
    q_lat = torch.randn(ctx, H, R, generator=g) * 0.2
    q_raw = torch.randn(ctx, H, dn + dr, generator=g) * 0.3
    lat = torch.randn(ctx, R, generator=g) * 0.5
    k_rot = torch.randn(ctx, dr, generator=g) * 0.3
    probes = []
    for n, r in enumerate([window + 5, window + BS + 1, ctx - 1,
                           ctx // 2 + 3, 3 * ctx // 4]):
        for hd, j in ((0, r - window + 1), (1, r - window), (2, r - 3)):
            # head hd of row r looks for key j along one axis
            axis = (3 * n + hd) % R
            lat[j] = 0
            lat[j, axis] = 4.0
            q_lat[r, hd] = 0
            q_lat[r, hd, axis] = 5.0
        probes.append(r)
    rows = sorted(set(probes + [0, 1, BS - 1, BS, window - 1, window]))
    q_lat, q_raw, lat, k_rot = (t.to(act) for t in (q_lat, q_raw, lat, k_rot))
    scale = 0.9
    pos = torch.arange(ctx)
    want = oracle.windowed_latent_rows(
        q_lat.double(),
        oracle.rotate_pairs(q_raw[..., dn:].double(), pos, dims, base),
        lat.double(), k_rot.double(), window, scale)
    # the dominating key really decides: inside the window it is nearly all
    # of the output, one place outside it is not
    r0 = probes[0]
    assert float(want[r0, 0].abs().max()) > 3.0
    assert float(want[r0, 1].abs().max()) < 3.0
    nb = -(-ctx // BS) + 3
    perm = torch.randperm(nb, generator=g).tolist()
    cache = torch.zeros(nb, 1, BS, R + dr, dtype=act)
    for p in range(ctx):
        cache[perm[p // BS], 0, p % BS] = torch.cat([lat[p], k_rot[p]])
    cache = cache.to(device)
    bt = _i32([perm[::-1], perm], device)
    cs = angle_table(ctx, dims, base).to(device)

    def run(rs, ps=None):
        n = len(rs)
        out = torch.full((H, n, R), 9.0, dtype=act, device=device)
        qa = q_lat[rs].permute(1, 0, 2).contiguous().to(device)
        qq = torch.zeros(n, H * (dn + dr) + 2, dtype=act)
        qq[:, : H * (dn + dr)] = q_raw[rs].reshape(n, -1)
        ops.latent_attention(out, qa, qq.to(device), cache, cs,
                             _i32(ps if ps is not None else rs, device),
                             _i32([1] * n, device), bt, H, dn, dr, window,
                             scale)
        return out.permute(1, 0, 2)

    _close(run(rows), want[rows], dtype, "prompt rows", scale=1.0)
    _close(run(list(range(ctx))), want, dtype, "every row", scale=1.0)
    _close(run(list(range(37, ctx))), want[37:], dtype, "a portion's rows",
           scale=1.0)
    for r in probes + [0, window]:
        _close(run([r]), want[[r]], dtype, f"decoded row {r}", scale=1.0)
    out = run(rows[:3], [rows[0], -1, rows[2]])
    assert float(out[1].abs().max()) == 0.0
    _close(out[[0, 2]], want[[rows[0], rows[2]]], dtype, "beside an inactive row",
           scale=1.0)
    # no window at all
    full = oracle.windowed_latent_rows(
        q_lat.double(),
        oracle.rotate_pairs(q_raw[..., dn:].double(), pos, dims, base),
        lat.double(), k_rot.double(), 0, scale)
    n = len(rows)
    o2 = torch.empty(H, n, R, dtype=act, device=device)
    qq = q_raw[rows].reshape(n, -1).to(device)
    ops.latent_attention(o2, q_lat[rows].permute(1, 0, 2).contiguous().to(device),
                         qq, cache, cs, _i32(rows, device),
                         _i32([1] * n, device), bt, H, dn, dr, 0, scale)
    _close(o2.permute(1, 0, 2), full[rows], dtype, "unbounded", scale=1.0)
