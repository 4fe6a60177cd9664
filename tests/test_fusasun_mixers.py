"""The Fusasun decoder's mechanisms, each alone, against the plain float64 implementations of
``fusasun_oracle``: the framework's mixers over a paged cache / state slots, whole sequences, cut into
portions and decoded token by token, on the CPU path and (``gpu`` marker) on the HIP kernels in f32 and
bf16.  Where random weights would hide a fault (a window's edge, a block that is just seen or not yet, a far
key) the weights and inputs are made so that it shows."""
import math

import pytest
import torch

import fusasun_oracle as O
from llm_kubernetes_minikube_sharp4dev_amd import ops
from llm_kubernetes_minikube_sharp4dev_amd.models import FusasunConfig, build_decoder
from llm_kubernetes_minikube_sharp4dev_amd.models.attention import AttnMeta
from llm_kubernetes_minikube_sharp4dev_amd.models.window_attention import RotarySpec

CPU32 = pytest.param("cpu", torch.float32, id="cpu-f32")
GPU32 = pytest.param("cuda", torch.float32, id="gpu-f32", marks=pytest.mark.gpu)
GPU16 = pytest.param("cuda", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)
ALL = [CPU32, GPU32, GPU16]
BS = 16


def tol(dtype):
    return 3e-5 if dtype == torch.float32 else 4e-2


def rel_err(got, want):
    want = want.double()
    return float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-9))


def rnd(g, *shape, scale=1.0):
    return torch.randn(*shape, generator=g, dtype=torch.float64) * scale


def q16(t):
    """Values a bf16 tensor holds exactly, so both sides of a comparison start from the same numbers."""
    return t.to(torch.bfloat16).to(torch.float64)


def step_meta(seqs, device):
    """AttnMeta of one step, as the model runner lays it out: ``seqs`` = [(start, n, block table, state
    slot, decode row?)], prompt portions first, then decode rows (n == 1)."""
    pre = [s for s in seqs if not s[4]]
    dec = [s for s in seqs if s[4]]
    pos, slots, cu, ctx_p, st = [], [], [0], [], []
    for start, n, table, slot, _ in pre + dec:
        for p in range(start, start + n):
            pos.append(p)
            slots.append(table[p // BS] * BS + p % BS)
        st.append(slot)
    for start, n, *_ in pre:
        cu.append(cu[-1] + n)
        ctx_p.append(start + n)
    i32 = dict(dtype=torch.int32, device=device)

    def tables(group):
        w = max(len(s[2]) for s in group)
        return torch.tensor([list(s[2]) + [0] * (w - len(s[2])) for s in group], **i32)

    m = AttnMeta(positions=torch.tensor(pos, **i32), slots=torch.tensor(slots, **i32), num_prefill_tokens=cu[-1],
                 num_prefill_seqs=len(pre), num_decode=len(dec))
    if pre:
        m.cu_q, m.ctx_lens_p, m.block_tables_p = torch.tensor(cu, **i32), torch.tensor(ctx_p, **i32), tables(pre)
        m.q_lens_cpu, m.ctx_lens_cpu = [s[1] for s in pre], ctx_p
    if dec:
        m.block_tables_d, m.ctx_lens_d = tables(dec), torch.tensor([s[0] + 1 for s in dec], **i32)
    lens = [s[1] for s in pre] + [1] * len(dec)
    m.seq_cu = torch.tensor([0] + [int(v) for v in torch.tensor(lens).cumsum(0)], **i32)
    m.state_slots = torch.tensor(st, **i32)
    m.max_seq_len = max(lens)
    return m


def one_layer(kind, mixer, W, device, dtype, seed=5, eps=1e-5, taps=3, sd=None):
    """A one-layer model of the mechanism (random weights through the checkpoint names, or ``sd``) and its tensors."""
    cfg = FusasunConfig.from_json({"architecture": "Fusasun", "vocab": 11, "width": W, "norm": {"eps": eps}, "embedding": {"scale": 1.0},
                                   "canon": {"taps": taps}, "layers": [{"type": kind, "mixer": mixer, "mlp": None}]})
    m = build_decoder(cfg, device=device, dtype=dtype, seed=seed)
    if sd is not None:
        full = {k: v.cpu() for k, v in m.native_state_dict().items()}
        full.update(sd)
        m.load_state_dict_native(full)
    out = {k: v.cpu().double() for k, v in m.native_state_dict().items()}
    return m, out


def run_mixer(m, h, cuts, device, dtype, slot=1, blocks=None, nblocks=40, caches=None):
    """The layer's mixer over ``h`` [T, W] fed in portions of the sizes ``cuts`` (the rest as decode rows)."""
    T = h.shape[0]
    blocks = blocks or list(range(nblocks - 1, nblocks - 1 - (T + BS - 1) // BS, -1))   # pages in descending order
    caches = caches or m.make_caches(nblocks, BS, 3)
    out, at, sizes = [], 0, list(cuts)
    while at < T:
        dec = not sizes
        n = 1 if dec else min(sizes.pop(0), T - at)
        meta = step_meta([(at, n, blocks, slot, dec)], device)
        with torch.inference_mode():
            y = m._mixer(m.layers[0], h[at:at + n].to(dtype).to(device).contiguous(), meta, caches[0])
        out.append(y.float().cpu())
        at += n
    return torch.cat(out)


def want_mixer(kind, h, mixer, sd, eps=1e-5):
    hc = O.canon(h, sd["l0.canon1"])
    if kind == "attention":
        return O.pooled_window_attention(hc, mixer, sd, "l0.mix.")
    return O.latent_window_attention(hc, mixer, sd, "l0.mix.", eps)


ATT = {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 16, "scale": 0.3, "mask": {"size": 13, "pool": 5},
       "rot": {"dims": 10, "base": 50.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 40}}}
LAT = {"heads": 3, "dim": 12, "rot_dim": 6, "vdim": 20, "q_rank": 14, "kv_rank": 18, "scale": 0.35, "mask": {"size": 11},
       "rot": {"dims": 6, "base": 30.0, "scaling": {"factor": 3.0, "original": 24, "fast": 4.0, "slow": 1.0}}}
KINDS = {"attention": ATT, "latent_attention": LAT}


def test_frequency_tables_of_both_scalings():
    """The frequency tables against the oracle's: bands (every band populated, also without scaling) and ramp
    (pairs before, inside and behind the ramp; the magnitude of cos and sin)."""
    for rot in (ATT["rot"], {"dims": 32, "base": 7000.0, "scaling": {"factor": 6.0, "low": 1.0, "high": 3.0, "original": 300}},
                {"dims": 8, "base": 100.0}):
        f, mag = RotarySpec.from_dict(rot, "bands").table()
        wf, wm = O.llama3_freqs(rot)
        assert mag == wm == 1.0 and f == pytest.approx(wf, rel=1e-14)
    plain = [50.0 ** (-2.0 * i / 10) for i in range(5)]
    f = RotarySpec.from_dict(ATT["rot"], "bands").table()[0]
    kinds = {("kept" if a == b else "divided" if abs(a - b / 4.0) < 1e-15 else "between") for a, b in zip(f, plain)}
    assert kinds == {"kept", "divided", "between"}
    for rot in (LAT["rot"], {"dims": 24, "base": 90000.0, "scaling": {"factor": 5.0, "original": 1000, "fast": 16.0, "slow": 2.0}},
                {"dims": 6, "base": 10.0}):
        f, mag = RotarySpec.from_dict(rot, "ramp").table()
        wf, wm = O.yarn_freqs(rot)
        assert mag == pytest.approx(wm, rel=1e-14) and f == pytest.approx(wf, rel=1e-14)
    assert RotarySpec.from_dict(LAT["rot"], "ramp").magnitude == pytest.approx(0.1 * math.log(3.0) + 1.0)


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("kind", list(KINDS))
def test_mixer_whole_portions_and_token_by_token(kind, device, dtype):
    """A whole prompt in one step, token by token from the first token on, and portions of 1, 2, 2, 3,
    16, 17, 5 tokens followed by decode rows give the oracle's result at every position (convolution state,
    window, pooled blocks and rotation all cross the cuts)."""
    mixer = KINDS[kind]
    W, T = 40, 61
    m, sd = one_layer(kind, mixer, W, device, dtype)
    h = q16(rnd(torch.Generator().manual_seed(3), T, W))
    want = want_mixer(kind, h, mixer, sd)
    for cuts in ([T], [1], [1, 2, 2, 3, 16, 17, 5], [30, 2, 29]):
        got = run_mixer(m, h, cuts, device, dtype)
        assert rel_err(got, want) < tol(dtype), (cuts, rel_err(got, want))


def _selector_weights(H, G, dim, vdim, W):
    """Projections that copy columns of the input: q = h[:, :H dim], k and v the next columns; no convolution;
    an output projection that copies the heads' results into the first columns."""
    eye = torch.eye(W)
    o = torch.zeros(W, H * vdim)
    o[:H * vdim] = torch.eye(H * vdim)
    return {"l0.mix.q": eye[:H * dim], "l0.mix.k": eye[H * dim:(H + G) * dim], "l0.mix.v": eye[(H + G) * dim:(H + G) * dim + G * vdim],
            "l0.mix.o": o, "l0.canon1": torch.zeros(W, 1)}


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("window,pool", [(13, 5), (16, 16), (32, 4), (7, 1), (20, 0)])
def test_window_and_block_edges_stand_out(window, pool, device, dtype):
    """One key (at position j0, in an unrotated dimension every query points along) outweighs all others by
    far, and its value is a marker.  A query then returns the marker while j0 is inside its window, nothing of
    it in the gap after the window has passed and before j0's block is seen, and -- through the block's mean
    key -- mostly the block's mean value from then on; queries and positions are checked on both sides of every
    edge, in one step, in portions and token by token."""
    H, G, dim, vdim = 2, 1, 8, 8
    W = H * dim + G * dim + G * vdim
    mask = {"size": window, "pool": pool} if pool else {"size": window}
    mixer = {"heads": H, "kv_heads": G, "dim": dim, "vdim": vdim, "scale": 1.0, "mask": mask, "rot": {"dims": 4, "base": 10.0}}
    m, sd = one_layer("attention", mixer, W, device, dtype, taps=1, sd=_selector_weights(H, G, dim, vdim, W))
    j0 = 12
    T = j0 + window + 3 * max(pool, 1) + 5
    g = torch.Generator().manual_seed(7)
    h = q16(rnd(g, T, W, scale=0.3))
    h[:, 7] = h[:, 15] = 2.0                    # both query heads point along the last (unrotated) dimension
    h[:, H * dim + 7] = 0.0
    h[j0, H * dim + 7] = 24.0 * max(pool, 1)    # so that also the block's mean key stands out
    h[j0, (H + G) * dim:] = 0.0
    h[j0, (H + G) * dim + 3] = 50.0             # the marker
    want = O.pooled_window_attention(h, mixer, sd, "l0.mix.")
    mark = want[:, 3]
    assert float(mark[j0 + window - 1]) > 45.0                      # last position that has j0 in its window
    first_seen = (j0 // pool) * pool + pool - 1 + window if pool else None      # the block's last position leaves the window
    gap = range(j0 + window, first_seen if pool else T)
    assert all(abs(float(mark[i])) < 1.0 for i in gap)              # out of the window, block not yet seen (or never)
    if pool:
        assert float(mark[first_seen]) > 40.0 / pool and (pool == 1 or first_seen > j0 + window)
    for cuts in ([T], [1], [j0 + window - 1, 1, 1, 2], [5, 2, 2, 16, 3]):
        got = run_mixer(m, h, cuts, device, dtype)
        assert rel_err(got, want) < tol(dtype), (cuts, rel_err(got, want))


@pytest.mark.parametrize("device,dtype", ALL)
def test_far_key_reaches_a_query_through_its_block_only(device, dtype):
    """A marked key 380 positions back, among hundreds, can reach a query only through the pooled entry of
    its block (window 30, blocks of 7): prompts in one step, in portions across pages, and decode rows, with
    two key splits' worth of pooled entries."""
    H, G, dim, vdim = 2, 1, 8, 8
    W = H * dim + G * dim + G * vdim
    mixer = {"heads": H, "kv_heads": G, "dim": dim, "vdim": vdim, "scale": 1.0, "mask": {"size": 30, "pool": 7},
             "rot": {"dims": 6, "base": 100.0, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 64}}}
    m, sd = one_layer("attention", mixer, W, device, dtype, taps=1, sd=_selector_weights(H, G, dim, vdim, W))
    T, j0 = 400, 17
    h = q16(rnd(torch.Generator().manual_seed(8), T, W, scale=0.3))
    h[:, 7] = h[:, 15] = 2.0
    h[:, H * dim + 7] = 0.0
    h[j0, H * dim + 7] = 7 * 30.0
    h[j0, (H + G) * dim:] = 0.0
    h[j0, (H + G) * dim + 3] = 70.0
    want = O.pooled_window_attention(h, mixer, sd, "l0.mix.")
    assert float(want[T - 1, 3]) > 9.0 and abs(float(want[j0 + 30, 3])) < 1.0
    for cuts in ([T], [350], [100, 37, 200, 2]):
        got = run_mixer(m, h, cuts, device, dtype)
        assert rel_err(got, want) < tol(dtype), (cuts, rel_err(got, want))


@pytest.mark.parametrize("device,dtype", ALL)
def test_long_window_with_blocks_behind_it(device, dtype):
    """A window of 520 positions (the prompt kernels then split a tile's keys over the waves of a workgroup
    instead of giving each wave a tile) with blocks of 8 behind it: one head, whole prompt, portions and decode
    rows across the position where the first blocks come into sight."""
    mixer = {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.5, "mask": {"size": 520, "pool": 8},
             "rot": {"dims": 8, "base": 1000.0, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 256}}}
    W, T = 24, 575
    m, sd = one_layer("attention", mixer, W, device, dtype, taps=2)
    h = q16(rnd(torch.Generator().manual_seed(12), T, W))
    want = want_mixer("attention", h, mixer, sd)
    for cuts in ([T], [526, 2, 40], [540]):
        got = run_mixer(m, h, cuts, device, dtype)
        assert rel_err(got, want) < tol(dtype), (cuts, rel_err(got, want))


@pytest.mark.parametrize("device,dtype", ALL)
def test_latent_window_edge_and_head_gate(device, dtype):
    """Latent attention with a window of 6: random weights, but the input of one position scaled up so that its
    key and value dominate while it is visible; positions on both sides of the window's edge, whole / portions /
    token by token."""
    mixer = dict(LAT, mask={"size": 6})
    W, T = 32, 40
    m, sd = one_layer("latent_attention", mixer, W, device, dtype, taps=2)
    h = q16(rnd(torch.Generator().manual_seed(9), T, W))
    h[20] *= 6.0
    want = want_mixer("latent_attention", h, mixer, sd)
    for cuts in ([T], [1], [21, 1, 4, 1, 1], [25, 2]):
        got = run_mixer(m, h, cuts, device, dtype)
        assert rel_err(got, want) < tol(dtype), (cuts, rel_err(got, want))


@pytest.mark.parametrize("device,dtype", ALL)
def test_used_pages_and_slots_do_not_leak(device, dtype):
    """Caches and convolution state left full of another sequence's large values: a new sequence in the same
    pages and slot (first row at position 0) gives the oracle's result; two sequences in one step."""
    W = 40
    for kind, mixer in KINDS.items():
        m, sd = one_layer(kind, mixer, W, device, dtype)
        caches = m.make_caches(12, BS, 3)
        for c in caches[0]:
            c.fill_(300.0)
        g = torch.Generator().manual_seed(11)
        ha, hb = q16(rnd(g, 37, W)), q16(rnd(g, 21, W))
        wa, wb = want_mixer(kind, ha, mixer, sd), want_mixer(kind, hb, mixer, sd)
        ta, tb = [5, 2, 9], [7, 1]
        dev = lambda t: t.to(dtype).to(device).contiguous()
        with torch.inference_mode():
            y1 = m._mixer(m.layers[0], dev(torch.cat([ha[:30], hb[:20]])), step_meta([(0, 30, ta, 2, False), (0, 20, tb, 0, False)], device), caches[0])
            y2 = m._mixer(m.layers[0], dev(torch.cat([ha[30:], hb[20:]])), step_meta([(30, 7, ta, 2, False), (20, 1, tb, 0, True)], device), caches[0])
        got_a = torch.cat([y1[:30], y2[:7]]).float().cpu()
        got_b = torch.cat([y1[30:], y2[7:]]).float().cpu()
        assert rel_err(got_a, wa) < tol(dtype) and rel_err(got_b, wb) < tol(dtype), kind


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("W,parts", [(36, 1), (48, 2), (50, 3), (1024, 2)])
def test_gated_stream_update_and_column_norm(W, parts, device, dtype):
    g = torch.Generator().manual_seed(W)
    T, eps = 9, 1e-5
    x, y, gate = rnd(g, T, W).float(), q16(rnd(g, T * parts, W)), q16(rnd(g, T, W))
    gb, wp, wn = rnd(g, W).float(), rnd(g, W).float() + 1, rnd(g, W).float() + 1
    v = y.view(T, parts, W).mean(1) * torch.sigmoid(gate + gb.double())
    wx = x.double() + O.rms(v, eps) * wp.double()
    wh = O.rms(wx, eps) * wn.double()
    xd = x.clone().to(device)
    d = lambda t: t.to(device)
    hd = ops.stream_gated_norm(xd, d(y.to(dtype)), d(gate.to(dtype)), d(gb), d(wp), d(wn), eps, dtype, parts=parts)
    assert rel_err(xd, wx) < 3e-6 and rel_err(hd, wh) < (3e-6 if dtype == torch.float32 else 1e-2)
    x2 = x.clone().to(device)
    assert ops.stream_gated_norm(x2, d(y.to(dtype)), d(gate.to(dtype)), d(gb), d(wp), None, eps, dtype, parts=parts) is None
    assert torch.equal(x2, xd)
    u = q16(rnd(g, T, W + 11))
    w = rnd(g, W - 3).float()
    got = ops.rms_cols(d(u.to(dtype)), 5, W - 3, d(w), eps)
    assert rel_err(got, O.rms(u[:, 5:W + 2], eps) * w.double()) < (3e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("W,ff,E,top,T", [(48, 20, 5, 2, 37), (36, 13, 1, 1, 5), (50, 24, 7, 3, 70), (256, 128, 8, 2, 130),
                                          (64, 40, 2, 2, 150), (72, 100, 3, 1, 333), (44, 12, 2, 2, 100), (64, 24, 2, 2, 300), (128, 128, 2, 1, 700), (192, 256, 3, 2, 600)])
def test_table_routed_experts(W, ff, E, top, T, device, dtype):
    """Experts by token id: every expert used, tokens that share none, widths the 16-byte loads do not divide, few and
    many pairs per expert (narrow and wide row tiles of the grouped products with ragged last tiles; with 128 pairs per
    expert and sizes the dense GEMM tiles, its grouped form)."""
    g = torch.Generator().manual_seed(E * 100 + top)
    V = 23
    sd = {}
    for j in range(E):
        sd.update({f"m.e{j}.gate": q16(rnd(g, ff, W, scale=W ** -0.5)), f"m.e{j}.up": q16(rnd(g, ff, W, scale=W ** -0.5)),
                   f"m.e{j}.down": q16(rnd(g, W, ff, scale=ff ** -0.5))})
    table = torch.rand(V, E, generator=g).argsort(1)[:, :top].to(torch.int32)
    sd["m.table"] = table
    ids = torch.randint(0, V, (T,), generator=g)
    h = q16(rnd(g, T, W))
    want = O.table_moe(h, ids, {"router": {"experts": E, "top": top}}, sd, "m.")
    ffp = -(-ff // 8) * 8
    gu, dn = torch.zeros(E, 2 * ffp, W, dtype=torch.float64), torch.zeros(E, W, ffp, dtype=torch.float64)
    for j in range(E):
        gu[j, :ff], gu[j, ffp:ffp + ff], dn[j, :, :ff] = sd[f"m.e{j}.gate"], sd[f"m.e{j}.up"], sd[f"m.e{j}.down"]
    d = lambda t: t.to(dtype).to(device)
    y = ops.table_experts(d(h), ids.to(torch.int32).to(device), table.to(device), d(gu), d(dn), top)
    got = y.float().view(T, top, W).mean(1)
    assert rel_err(got, want) < (3e-5 if dtype == torch.float32 else 3e-2)
    seg, order = ops.moe_route(ids.to(torch.int32).to(device), table.to(device), E)
    e_of = table[ids.long()].reshape(-1)
    assert sorted(order.tolist()) == list(range(T * top)) and seg.tolist()[0] == 0 and seg.tolist()[-1] == T * top
    for e in range(E):
        assert all(int(e_of[p]) == e for p in order[int(seg[e]):int(seg[e + 1])].tolist())


@pytest.mark.parametrize("device,dtype", ALL)
@pytest.mark.parametrize("taps,W", [(1, 36), (3, 48), (4, 40), (8, 50)])
def test_convolution_added_to_its_input_over_cuts(taps, W, device, dtype):
    """h + conv(h) as one convolution whose last tap carries the identity, its state kept per slot across
    portions of 1, 2 and more tokens; the first tokens of a sequence see zeros before its start."""
    g = torch.Generator().manual_seed(taps)
    T = 29
    h, w = q16(rnd(g, T, W)), q16(rnd(g, W, taps, scale=0.5))
    want = O.canon(h, w)
    wf = w.float().clone()
    wf[:, -1] += 1.0
    state = torch.full((3, max(taps - 1, 1), W), 77.0, dtype=dtype, device=device)
    i32 = dict(dtype=torch.int32, device=device)
    out, at = [], 0
    for n in (1, 2, 1, 7, 2, 16):
        cu, sl, pos = torch.tensor([0, n], **i32), torch.tensor([2], **i32), torch.arange(at, at + n, **i32)
        out.append(ops.conv_silu(h[at:at + n].to(dtype).to(device).contiguous(), 0, W, wf.to(device), None, state, cu, sl, pos, n, act=False))
        at += n
    assert rel_err(torch.cat(out).float(), want) < (3e-6 if dtype == torch.float32 else 1e-2)
