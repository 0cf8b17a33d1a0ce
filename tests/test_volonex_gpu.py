"""Volonex on the GPU against the plain implementation (tests/plain/volonex_plain.py): each new
mechanism alone at the kernel, with keys planted so that a wrong edge, a lost sink or a far key
left out shows; then whole models of several shapes through the engine's step function, cut and
batched in many ways, in 32-bit and in bfloat16; and greedy generation through the library's own
entry point."""
import math

import pytest
import torch

from tests.helpers import argmax_agrees_where_clear, close, rand_ids
from tests.plain import volonex_plain as P
from tests.test_kernels_gpu import dev, fill_cache, paged_setup, rnd, cached_k, cached_v

pytestmark = pytest.mark.gpu
PAGE = 64
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def ops():
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.kernels import ops as o
    return o


# ------------------------------------------------------------------ small mechanisms
@pytest.mark.parametrize("dtype,wdtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                          (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("rows,D", [(5, 48), (3, 37), (70, 1000)])
def test_dynamic_tanh_with_the_scaled_residual_add(ops, dtype, wdtype, rows, D):
    resid = rnd(rows, D, seed=1, scale=2.0)
    delta = rnd(rows, D, seed=2).to(dtype)
    w, b = (1 + 0.3 * rnd(D, seed=3)).to(wdtype), rnd(D, seed=4).to(wdtype)
    alpha = torch.tensor(0.7).to(wdtype)
    r = dev(resid.clone())
    out = torch.empty(rows, D, dtype=dtype, device="cuda")
    ops.add_dyt(r, dev(delta), dev(w), dev(b), dev(alpha), out, rows, 0.35)
    new = resid.double() + 0.35 * delta.double()
    assert torch.allclose(r.cpu().double(), new, rtol=1e-6, atol=1e-6)
    want = P.dynamic_tanh(new, w.double(), b.double(), alpha.double())
    tol = 2e-6 if dtype == torch.float32 else 2 ** -7
    assert torch.allclose(out.cpu().double(), want, rtol=tol, atol=tol)
    # without a pending add the stream is left alone, and without an output only the add happens
    r2 = dev(resid.clone())
    ops.add_dyt(r2, None, dev(w), dev(b), dev(alpha), out, rows)
    assert torch.equal(r2.cpu(), resid)
    assert torch.allclose(out.cpu().double(), P.dynamic_tanh(resid.double(), w.double(), b.double(), alpha.double()),
                          rtol=tol, atol=tol)
    ops.add_dyt(r2, dev(delta), dev(w), dev(b), dev(alpha), None, rows)
    assert torch.allclose(r2.cpu().double(), resid.double() + delta.double(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,I,interleaved", [(3, 40, True), (9, 37, False), (65, 256, True)])
def test_bounded_gated_activation(ops, dtype, rows, I, interleaved):
    g, u = rnd(rows, I, seed=5, scale=3.0).to(dtype), rnd(rows, I, seed=6, scale=3.0).to(dtype)   # well beyond the limit
    x = torch.stack([g, u], 2).reshape(rows, 2 * I) if interleaved else torch.cat([g, u], 1)
    out = torch.empty(rows, I, dtype=dtype, device="cuda")
    ops.silu_mul(out, dev(x.contiguous()), rows, interleaved, alpha=1.702, limit=1.25, up_shift=1.0)
    gd, ud = g.double().clamp(max=1.25), u.double().clamp(-1.25, 1.25)
    want = gd * torch.sigmoid(1.702 * gd) * (ud + 1)
    tol = 2e-6 if dtype == torch.float32 else 2 ** -7
    assert torch.allclose(out.cpu().double(), want, rtol=tol, atol=tol)
    assert (g.double() > 1.25).any() and (u.double() < -1.25).any()      # the bounds were met


@pytest.mark.parametrize("M", [1, 8, 16, 20, 40, 64])
@pytest.mark.parametrize("I,K", [(160, 264), (1008, 520)])
def test_bounded_gated_activation_as_the_epilogue_of_a_product(ops, M, I, K):
    x = rnd(M, K, seed=11).to(torch.bfloat16)
    g, u = (rnd(I, K, seed=12) * 0.2).to(torch.bfloat16), (rnd(I, K, seed=13) * 0.2).to(torch.bfloat16)
    w = torch.stack([g, u], 1).reshape(2 * I, K).contiguous()        # gate i at row 2i, its up at 2i + 1
    out = torch.empty(M, I, dtype=torch.bfloat16, device="cuda")
    act = (1.702, 0.75, 1.0)
    if M <= 16:
        ops.gemm_blocksplit(out, dev(x), dev(w), None, M, gated=True, act=act)
    else:
        ops.gemm_rows(out, None, dev(x), dev(w), None, M, gated=True, plan=(0, 0, 1), act=act)
    gd = (x.double() @ g.double().T).clamp(max=0.75)
    ud = (x.double() @ u.double().T).clamp(-0.75, 0.75)
    assert (x.double() @ g.double().T > 0.75).any()
    want = gd * torch.sigmoid(1.702 * gd) * (ud + 1)
    assert torch.allclose(out.cpu().double(), want, rtol=2 ** -7, atol=2 ** -7)


def test_embedding_scale_and_scaled_residual_add(ops):
    table = rnd(50, 24, seed=7).to(torch.bfloat16)
    ids = torch.tensor([3, 49, 0, 7], dtype=torch.int32)
    out = torch.empty(4, 24, device="cuda")
    ops.embedding(out, dev(table), dev(ids), 4, 5.5)
    assert torch.allclose(out.cpu().double(), table[ids.long()].double() * 5.5, rtol=1e-6)
    r = rnd(4, 24, seed=8)
    d = rnd(4, 24, seed=9)
    rr = dev(r.clone())
    ops.residual_add(rr, dev(d), 4, 0.25)
    assert torch.allclose(rr.cpu().double(), r.double() + 0.25 * d.double(), rtol=1e-6, atol=1e-7)


ROTS = [
    {"base": 10000.0, "dims": 16, "scaling": {"factor": 8.0, "original": 64, "fast": 8.0, "slow": 2.0}},
    {"base": 500.0, "dims": 24},
    {"base": 1000000.0, "dims": 8, "scaling": {"factor": 2.5, "original": 4096, "fast": 64.0, "slow": 0.5}},
]


@pytest.mark.parametrize("rot", ROTS)
def test_rotary_frequencies_of_the_part_equal_the_plain_ones(rot):
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.parts.base import BuildEnv, PartSpec, build_part
    params = {"head_dim": 32, "rotary_dim": rot["dims"], "theta": rot["base"], "interleaved": True}
    if "scaling" in rot:
        params["scaling"] = {"kind": "yarn", **rot["scaling"]}
    part = build_part("position", PartSpec("rotary", params), "x.", BuildEnv(torch.device("cuda"), torch.float32))
    f, mult = P.rotary_frequencies(rot)
    assert torch.allclose(part.rotary()[0].cpu().double(), f, rtol=1e-7)
    assert abs(part.mscale - mult) < 1e-12 and part.interleaved
    if "scaling" in rot:        # the ramp really lies inside: some frequencies scaled, some not
        plain, _ = P.rotary_frequencies({"base": rot["base"], "dims": rot["dims"]})
        assert (f == plain).any() or rot["dims"] == 8
        assert (f < plain * 0.999).any()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KVH,kd,vd,pd,rot", [(4, 2, 32, 16, 32, ROTS[0]), (3, 1, 24, 40, 48, ROTS[1]),
                                                (2, 2, 16, 16, 16, ROTS[2]), (2, 1, 40, 40, 48, None)])
def test_interleaved_rotation_and_cache_write_into_padded_heads(ops, dtype, H, KVH, kd, vd, pd, rot):
    starts, new = [70, 5000, 0], [3, 66, 1]
    slots, table, kpool, vpool = paged_setup([a + b for a, b in zip(starts, new)], KVH, pd, dtype, 31)
    rows = sum(new)
    width = H * kd + KVH * kd + KVH * vd + H          # gate columns ride along and are left alone
    qkv = rnd(rows, width, seed=32).to(dtype)
    positions = torch.cat([torch.arange(a, a + b) for a, b in zip(starts, new)]).int()
    row_seq = torch.cat([torch.full((b,), i) for i, b in enumerate(new)]).int()
    f, mult = P.rotary_frequencies(rot) if rot else (None, 1.0)
    r = rot["dims"] if rot else 0
    q_out = torch.full((rows, H * pd), 9.0, dtype=dtype, device="cuda")
    kp, vp = dev(kpool), dev(vpool)
    ops.qkv_rope_cache(q_out, kp, vp, dev(qkv), H * kd, KVH * kd, None, dev(positions), dev(row_seq),
                       dev(torch.tensor(slots, dtype=torch.int32)), dev(table),
                       dev(f.float()) if rot else None, r, rows, H, KVH, pd, True,
                       key_dim=kd, value_dim=vd, interleaved=True, mscale=mult)
    x = qkv.double()
    q = P.rotate_interleaved(x[:, :H * kd].reshape(rows, H, kd), positions.tolist(), rot, single=True)
    k = P.rotate_interleaved(x[:, H * kd:(H + KVH) * kd].reshape(rows, KVH, kd), positions.tolist(), rot, single=True)
    v = x[:, (H + KVH) * kd:(H + KVH) * kd + KVH * vd].reshape(rows, KVH, vd)
    tol = 2e-5 if dtype == torch.float32 else 2 ** -7
    got_q = q_out.cpu().double().reshape(rows, H, pd)
    assert torch.allclose(got_q[:, :, :kd], q, rtol=tol, atol=tol * 4)
    assert got_q[:, :, kd:].abs().max().item() == 0 if pd > kd else True        # the padding is zeros
    kp, vp = kp.cpu(), vp.cpu()
    for i in range(rows):
        page = table[slots[row_seq[i]], positions[i] // PAGE].item()
        ck, cv = cached_k(kp, page, positions[i] % PAGE, pd).double(), cached_v(vp, page, positions[i] % PAGE, pd).double()
        assert torch.allclose(ck[:, :kd], k[i], rtol=tol, atol=tol * 4) and ck[:, kd:].abs().sum() == 0
        assert torch.allclose(cv[:, :vd], v[i], rtol=tol, atol=tol * 4) and cv[:, vd:].abs().sum() == 0


# ------------------------------------------------------------------ attention kernels
def plain_attention(q, k, v, q_pos, chunk, window, scale, sinks, gate):
    """q [m, H, d], k/v [n, KVH, d] at positions 0..n-1; the design's attention, key by key."""
    m, H, d = q.shape
    G = k.shape[1]
    out = torch.zeros(m, H, v.shape[2], dtype=torch.float64)
    for t, p in enumerate(q_pos):
        js = [j for j in range(k.shape[0]) if P.sees(p, j, chunk, window)]
        for h in range(H):
            kv = h // (H // G)
            s = (k[js, kv] @ q[t, h]) * scale
            a = P.softmax_with_sink(s, sinks[h]) if sinks is not None else torch.softmax(s, 0)
            out[t, h] = (a @ v[js, kv]) * (torch.sigmoid(gate[t, h]) if gate is not None else 1.0)
    return out


def run_attention(ops, kind, dtype, H, KVH, hd, chunk, window, lengths, q_lens, seed, sinks=True, gated=True,
                  plant=None, tiles=0, parts=1):
    B = len(lengths)
    slots, table, kpool, vpool = paged_setup(lengths, KVH, hd, dtype, seed)
    ks = [rnd(n, KVH, hd, seed=seed + 10 + i).to(dtype) for i, n in enumerate(lengths)]
    vs = [rnd(n, KVH, hd, seed=seed + 20 + i).to(dtype) for i, n in enumerate(lengths)]
    qs = [rnd(m, H, hd, seed=seed + 30 + i, scale=2.0).to(dtype) for i, m in enumerate(q_lens)]
    if plant is not None:
        plant(qs, ks, vs)
    fill_cache(table, slots, kpool, vpool, ks, vs)
    rows = sum(q_lens)
    q = torch.cat(qs).reshape(rows, H * hd)
    positions = torch.cat([torch.arange(n - m, n) for n, m in zip(lengths, q_lens)]).int()
    row_seq = torch.cat([torch.full((m,), i) for i, m in enumerate(q_lens)]).int()
    cu = torch.tensor([0] + torch.tensor(q_lens).cumsum(0).tolist(), dtype=torch.int32)
    seq_start = torch.tensor([n - m for n, m in zip(lengths, q_lens)], dtype=torch.int32)
    seq_slot = torch.tensor(slots, dtype=torch.int32)
    sink = (rnd(H, seed=seed + 40, scale=2.0) + 1.0).to(dtype) if sinks else None
    # the gates lie inside a wider buffer, as they do behind q||k||v
    gbuf = rnd(rows, H + 5, seed=seed + 41, scale=2.0).to(dtype) if gated else None
    gd = dev(gbuf) if gated else None
    gate = gd[:, 3:3 + H] if gated else None
    out = torch.full((rows, H * hd), 7.0, dtype=dtype, device="cuda")
    scale = 0.9 / math.sqrt(hd)
    kw = dict(chunk=chunk, sinks=dev(sink) if sinks else None, gate=gate)
    args = (dev(kpool), dev(vpool))
    if kind == "plain":
        ops.attention_plain(out, dev(q), *args, dev(positions), dev(row_seq), dev(seq_slot), dev(table), rows,
                            H, KVH, hd, window, scale, **kw)
        most = max(lengths) + 3
        floats = ops.attention_plain_workspace_floats(rows, H, hd, most, window, chunk)
        if floats:      # page by page in parallel: the same bits
            again = torch.full((rows, H * hd), 7.0, dtype=dtype, device="cuda")
            ops.attention_plain(again, dev(q), *args, dev(positions), dev(row_seq), dev(seq_slot), dev(table),
                                rows, H, KVH, hd, window, scale, most, torch.empty(floats, device="cuda"), **kw)
            assert torch.equal(again, out)
    elif kind == "decode":
        ws = torch.empty(ops.attention_decode_workspace_floats(rows, H, KVH, hd, 4096), device="cuda")
        ops.attention_decode(out, dev(q), *args, dev(positions), dev(row_seq), dev(seq_slot), dev(table), rows,
                             H, KVH, hd, window, scale, 4096, ws, **kw)
    else:
        ws = torch.empty(ops.attention_prefill_workspace_floats(rows, H, hd, parts), device="cuda") if parts > 1 else None
        ops.attention_prefill(out, dev(q), *args, dev(cu), dev(seq_slot), dev(seq_start), dev(table), B,
                              max(q_lens), rows, H, KVH, hd, window, scale, kernel=tiles, parts=parts,
                              workspace=ws, **kw)
    got, want = [], []
    r = 0
    for i, (n, m) in enumerate(zip(lengths, q_lens)):
        got.append(out.cpu()[r:r + m].double().reshape(m, H, hd))
        want.append(plain_attention(qs[i].double(), ks[i].double(), vs[i].double(), list(range(n - m, n)), chunk,
                                    window, scale, sink.double() if sinks else None,
                                    gbuf[r:r + m, 3:3 + H].double() if gated else None))
        r += m
    return got, want


def same(got, want, dtype):
    tol = 4e-6 if dtype == torch.float32 else 2 ** -6
    for g, w in zip(got, want):
        assert torch.allclose(g, w, rtol=tol, atol=tol), (g - w).abs().max().item()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KVH,hd", [(6, 3, 48), (4, 1, 64), (5, 5, 16), (2, 1, 80)])
@pytest.mark.parametrize("chunk,window", [(24, 0), (64, 0), (70, 0), (100, 30), (0, 0)])
def test_plain_attention_with_chunks_sinks_and_gates(ops, dtype, H, KVH, hd, chunk, window):
    got, want = run_attention(ops, "plain", dtype, H, KVH, hd, chunk, window, [200, 3, 141], [7, 3, 80], 50)
    same(got, want, dtype)
    got, want = run_attention(ops, "plain", dtype, H, KVH, hd, chunk, window, [130, 71], [1, 1], 51, sinks=False)
    same(got, want, dtype)


@pytest.mark.parametrize("H,KVH,hd", [(6, 3, 48), (4, 1, 64), (28, 4, 128), (40, 2, 32), (2, 1, 256)])
@pytest.mark.parametrize("chunk,window", [(24, 0), (64, 0), (70, 0), (100, 30), (0, 0)])
def test_one_token_attention_with_chunks_sinks_and_gates(ops, H, KVH, hd, chunk, window):
    # lengths whose last position is the first of a chunk, the last of one, and in between
    lengths = [1, 25, 64, 65, 141, 200, 700]
    got, want = run_attention(ops, "decode", torch.bfloat16, H, KVH, hd, chunk, window, lengths, [1] * len(lengths), 60)
    same(got, want, torch.bfloat16)
    got, want = run_attention(ops, "decode", torch.bfloat16, H, KVH, hd, chunk, window, [300], [1], 61, gated=False)
    same(got, want, torch.bfloat16)


@pytest.mark.parametrize("H,KVH,hd", [(6, 3, 48), (4, 1, 64), (7, 1, 128), (2, 1, 192)])
@pytest.mark.parametrize("chunk,window", [(24, 0), (64, 0), (70, 0), (100, 30), (200, 0)])
@pytest.mark.parametrize("tiles", [0, 1])
def test_prompt_attention_with_chunks_sinks_and_gates(ops, H, KVH, hd, chunk, window, tiles):
    if tiles == 0 and hd > 128:
        tiles = 1
    # whole prompts, a continuation that starts inside a chunk, one that starts at a chunk's first position
    starts = [0, 0, 37, chunk * 3]
    q_lens = [300, 5, 150, 131]
    got, want = run_attention(ops, "prefill", torch.bfloat16, H, KVH, hd, chunk, window,
                              [a + b for a, b in zip(starts, q_lens)], q_lens, 70, tiles=tiles)
    same(got, want, torch.bfloat16)


@pytest.mark.parametrize("parts", [2, 5])
@pytest.mark.parametrize("chunk", [0, 300])
def test_prompt_attention_in_parts_joins_the_sink_once(ops, parts, chunk):
    got, want = run_attention(ops, "prefill", torch.bfloat16, 4, 2, 64, chunk, 0, [900, 700], [20, 9], 80, parts=parts)
    same(got, want, torch.bfloat16)


@pytest.mark.parametrize("kind", ["plain32", "plain", "decode", "prefill"])
@pytest.mark.parametrize("where", ["just_outside", "first_of_chunk", "far_inside", "own_key"])
def test_a_planted_key_at_the_edge_of_a_chunk(ops, kind, where):
    """One key answers the last query so strongly that it takes nearly all the weight: whether it
    counts decides the output. Its value is unlike every other."""
    dtype = torch.float32 if kind == "plain32" else torch.bfloat16
    H, KVH, hd, chunk, n = 4, 2, 32, 48, 48 * 5 + 20           # the last query sits at 259, its chunk starts at 240
    start = (n - 1) // chunk * chunk
    at = {"just_outside": start - 1, "first_of_chunk": start, "far_inside": start + 1, "own_key": n - 1}[where]

    def plant(qs, ks, vs):
        direction = torch.ones(hd) / math.sqrt(hd)
        qs[0][-1] = (direction * 40).to(dtype)
        ks[0][at] = (direction * 40).to(dtype)
        vs[0][at] = torch.full((KVH, hd), 25.0).to(dtype)

    q_lens = [1] if kind == "decode" else [n] if kind == "prefill" else [3]
    got, want = run_attention(ops, kind.replace("32", ""), dtype, H, KVH, hd, chunk, 0, [n], q_lens, 90, plant=plant)
    same(got, want, dtype)
    seen = want[0][-1].abs().max().item() > 5
    assert seen == (where != "just_outside")


@pytest.mark.parametrize("kind", ["plain32", "plain", "decode", "prefill"])
@pytest.mark.parametrize("at", [3, 63, 64, 640])
@pytest.mark.parametrize("chunk", [0, 1024])
def test_a_planted_key_far_back_among_hundreds(ops, kind, at, chunk):
    """The last query's answer lies hundreds of keys back (near the start, on either side of a page
    border, ten pages in): a kernel that drops a slice, a part or a page of the keys loses it."""
    dtype = torch.float32 if kind == "plain32" else torch.bfloat16
    H, KVH, hd, n = 6, 3, 48, 900

    def plant(qs, ks, vs):
        direction = torch.ones(hd) / math.sqrt(hd)
        qs[0][-1] = (direction * 40).to(dtype)
        ks[0][at] = (direction * 40).to(dtype)
        vs[0][at] = torch.full((KVH, hd), 25.0).to(dtype)

    q_lens = [1] if kind == "decode" else [n] if kind == "prefill" else [2]
    got, want = run_attention(ops, kind.replace("32", ""), dtype, H, KVH, hd, chunk, 0, [n], q_lens, 95, plant=plant)
    same(got, want, dtype)
    assert want[0][-1].abs().max().item() > 5


@pytest.mark.parametrize("kind", ["plain", "decode", "prefill"])
def test_a_large_sink_takes_the_weight_away(ops, kind):
    """A sink far above every score leaves almost nothing for the keys: a kernel that forgot it
    would return values of ordinary size."""
    H, KVH, hd = 4, 4, 32
    for n in (5, 140):
        slots, table, kpool, vpool = paged_setup([n], KVH, hd, torch.bfloat16, 3)
        ks, vs = [rnd(n, KVH, hd, seed=4).to(torch.bfloat16)], [rnd(n, KVH, hd, seed=5).to(torch.bfloat16) + 3]
        fill_cache(table, slots, kpool, vpool, ks, vs)
        m = 1 if kind == "decode" else n
        q = rnd(m, H * hd, seed=6).to(torch.bfloat16)
        sinks = torch.tensor([30.0, -30.0, 30.0, 0.0]).to(torch.bfloat16)
        pos = torch.arange(n - m, n).int()
        out = torch.empty(m, H * hd, dtype=torch.bfloat16, device="cuda")
        common = (dev(kpool), dev(vpool))
        zeros, slot = dev(torch.zeros(m, dtype=torch.int32)), dev(torch.tensor(slots, dtype=torch.int32))
        if kind == "plain":
            ops.attention_plain(out, dev(q), *common, dev(pos), zeros, slot, dev(table), m, H, KVH, hd, 0, 0.1,
                                sinks=dev(sinks))
        elif kind == "decode":
            ws = torch.empty(ops.attention_decode_workspace_floats(m, H, KVH, hd, 512), device="cuda")
            ops.attention_decode(out, dev(q), *common, dev(pos), zeros, slot, dev(table), m, H, KVH, hd, 0, 0.1,
                                 512, ws, sinks=dev(sinks))
        else:
            ops.attention_prefill(out, dev(q), *common, dev(torch.tensor([0, m], dtype=torch.int32)), slot,
                                  dev(torch.zeros(1, dtype=torch.int32)), dev(table), 1, m, m, H, KVH, hd, 0, 0.1,
                                  sinks=dev(sinks))
        o = out.cpu().double().reshape(m, H, hd)
        assert o[:, 0].abs().max() < 1e-6 and o[:, 2].abs().max() < 1e-6        # the sink took it all
        assert o[:, 1].abs().mean() > 1 and o[:, 3].abs().mean() > 0.5          # these heads kept theirs


# ------------------------------------------------------------------ whole models
def attn(heads, kv, dim, vdim, scale, chunk=None, rot=None):
    m = {"dim": dim, "heads": heads, "kv_heads": kv, "scale": scale, "vdim": vdim}
    if chunk:
        m["mask"] = {"size": chunk}
    if rot:
        m["rot"] = rot
    return m


def layer(mixer, ff=None, limit=None):
    return {"type": "attention", "mixer": mixer, "mlp": None if ff is None else {"ff": ff, "kind": "dense", "limit": limit}}


MODELS = {
    # keys wider than values and the other way round, a chunk smaller than a page and one that straddles pages,
    # a layer without a feed-forward, the first layer three times
    "V1": {"architecture": "Volonex", "vocab": 211, "width": 48, "residual_mult": 0.7, "embedding": {"scale": 3.0},
           "norm": {"eps": 1e-6}, "loop": {"start": 0, "stop": 1, "times": 3},
           "layers": [layer(attn(4, 2, 32, 16, 0.2, 24, ROTS[0]), 72, 1.5),
                      layer(attn(2, 1, 16, 48, 0.3, 70, {"base": 500.0, "dims": 16}))]},
    # equal widths, as many kv heads as heads, multiplier and scale 1, layers with no chunk and with no
    # rotation, the last two layers twice, a limit that hardly ever binds
    "V2": {"architecture": "Volonex", "vocab": 130, "width": 64, "residual_mult": 1.0, "embedding": {"scale": 1.0},
           "norm": {"eps": 1e-5}, "loop": {"start": 1, "stop": 3, "times": 2},
           "layers": [layer(attn(4, 4, 16, 16, 0.25, 16, ROTS[2]), 96, 7.0),
                      layer(attn(4, 4, 16, 16, 0.25, None, {"base": 10000.0, "dims": 4}), 40, 0.5),
                      layer(attn(2, 2, 32, 32, 0.17, 128), 64, 1.0)]},
    # head sizes that are no multiple of 16, a group of three, no loop at all, a chunk of 100
    "V3": {"architecture": "Volonex", "vocab": 97, "width": 40, "residual_mult": 0.4, "embedding": {"scale": 6.3},
           "norm": {"eps": 1e-6},
           "layers": [layer(attn(6, 2, 24, 40, 0.2, 100, ROTS[1]), 56, 2.0),
                      layer(attn(3, 3, 8, 8, 0.35, 33, {"base": 100.0, "dims": 8}), 24, 1.0)]},
}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """name -> model folder; the q and k matrices are made larger than the random default so that
    the attention weights are far from uniform and a key that is wrongly seen or missed matters."""
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.registry import config_from_dict
    from hector_engine_amd.weights import write_random_model
    from hector_engine_amd.weights.safetensors_io import write_safetensors
    from safetensors.torch import load_file
    out = {}
    for i, (name, cfg) in enumerate(MODELS.items()):
        folder = str(tmp_path_factory.mktemp(f"volonex_{name}"))
        write_random_model(config_from_dict(cfg), 40 + i, folder, "bfloat16")
        path = folder + "/model.safetensors"
        tensors = load_file(path)
        for k in tensors:
            if k.endswith(".mix.q") or k.endswith(".mix.k"):
                tensors[k] = (tensors[k].float() * 12).to(torch.bfloat16)
            elif k.endswith(".alpha") or k == "embed":
                pass
            elif tensors[k].dim() == 2:
                tensors[k] = (tensors[k].float() * 4).to(torch.bfloat16)
        write_safetensors(path, tensors, {"format": "pt"})
        out[name] = folder
    return out


@pytest.fixture(scope="module")
def plain(folders):
    return {name: P.read_model(f) for name, f in folders.items()}


@pytest.fixture(scope="module")
def engines(folders):
    import hector_engine_amd as he
    cache = {}

    def get(name, dtype, **kw):
        key = (name, dtype, tuple(sorted(kw.items())))
        if key not in cache:
            opts = dict(max_tokens=4096, max_slots=8, max_seq_len=1024)
            opts.update(kw)
            cache[key] = he.Engine(folders[name], dtype=dtype, **opts)
        return cache[key]

    return get


def entry(slot, tokens, want):
    from hector_engine_amd.engine.engine import StepEntry
    return StepEntry(slot, list(tokens), list(want))


def test_the_folder_written_from_a_configuration_reads_back(folders):
    import json
    from hector_engine_amd.registry import load_config
    for name, folder in folders.items():
        cfg = load_config(folder)
        assert cfg.to_dict() == json.load(open(folder + "/config.json"))
        assert [l for l, _ in cfg.runs()] == [l for l, _ in P.runs(MODELS[name])]
        assert [a for _, a in cfg.runs()] == [a for _, a in P.runs(MODELS[name])]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_each_request_alone_and_whole(engines, plain, name, dtype):
    eng = engines(name, dtype)
    cfg, w = plain[name]
    for seed, n in enumerate([1, 2, 23, 64, 65, 150]):
        ids = rand_ids(cfg["vocab"], n, seed)
        s = eng.acquire()
        got = eng.step([entry(s, ids, range(n))])
        want = P.forward(cfg, w, ids)
        close(got, want, dtype)
        argmax_agrees_where_clear(got, want, 0.05 * want.abs().max().item())
        eng.release(s)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_prompt_then_token_by_token_over_chunk_and_page_edges(engines, plain, name, dtype):
    eng = engines(name, dtype)
    cfg, w = plain[name]
    n, tail = 210, 150                  # the decoded positions 60..209 cross pages and every chunk size
    ids = rand_ids(cfg["vocab"], n, 11)
    want = P.forward(cfg, w, ids)
    s = eng.acquire()
    whole = eng.step([entry(s, ids, range(n))]).clone()
    eng.release(s)
    s = eng.acquire()
    assert eng.step([entry(s, ids[:n - tail], [])]) is None
    dec = torch.cat([eng.step([entry(s, [t], [0])]).clone() for t in ids[n - tail:]])
    eng.release(s)
    close(dec, want[n - tail:], dtype)
    if dtype == "float32":
        assert torch.equal(dec, whole[n - tail:])        # the 32-bit path does not depend on the cut
    else:
        close(dec, whole[n - tail:].cpu(), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
@pytest.mark.parametrize("cuts", [[2] * 40, [3, 2, 61, 17, 64, 2, 70], [1, 23, 24, 1, 25, 47, 48, 2], [128, 2, 2, 65]])
def test_prompts_fed_in_portions(engines, plain, name, dtype, cuts):
    eng = engines(name, dtype)
    cfg, w = plain[name]
    n = sum(cuts)
    ids = rand_ids(cfg["vocab"], n, 12)
    want = P.forward(cfg, w, ids)
    s = eng.acquire()
    whole = eng.step([entry(s, ids, range(n))]).clone()
    eng.release(s)
    s = eng.acquire()
    parts, at = [], 0
    for c in cuts:
        parts.append(eng.step([entry(s, ids[at:at + c], range(c))]).clone())
        at += c
    eng.release(s)
    got = torch.cat(parts)
    close(got, want, dtype)
    if dtype == "float32":
        assert torch.equal(got, whole)
    else:
        close(got, whole.cpu(), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_unequal_batches_equal_each_request_alone_and_slots_are_used_again(engines, plain, name, dtype):
    eng = engines(name, dtype, max_slots=4)
    cfg, w = plain[name]
    free = eng.cache.free_pages
    for round_no, lengths in enumerate([[1, 67, 140, 25], [90, 3, 49], [200, 2, 2, 64]]):
        prompts = [rand_ids(cfg["vocab"], n, 20 * round_no + i) for i, n in enumerate(lengths)]
        decode = 12
        full = [p + rand_ids(cfg["vocab"], decode - i, 500 + i) for i, p in enumerate(prompts)]   # shorter ones end earlier
        want = [P.forward(cfg, w, f) for f in full]
        slots = [eng.acquire() for _ in prompts]
        got = [[] for _ in prompts]
        logits = eng.step([entry(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)])
        for i in range(len(prompts)):
            got[i].append(logits[i:i + 1].clone())
        live = list(range(len(prompts)))
        for t in range(decode):
            live = [i for i in live if len(prompts[i]) + t < len(full[i])]
            if not live:
                break
            logits = eng.step([entry(slots[i], [full[i][len(prompts[i]) + t]], [0]) for i in live])
            for j, i in enumerate(live):
                got[i].append(logits[j:j + 1].clone())
        for i, s in enumerate(slots):
            eng.release(s)
            close(torch.cat(got[i]), want[i][len(prompts[i]) - 1:], dtype)
    assert eng.cache.free_pages == free


@pytest.mark.parametrize("name", list(MODELS))
def test_a_mixed_step_of_a_prompt_and_decoding_requests(engines, plain, name):
    eng = engines(name, "float32")
    cfg, w = plain[name]
    a, b = rand_ids(cfg["vocab"], 80, 30), rand_ids(cfg["vocab"], 37, 31)
    sa, sb = eng.acquire(), eng.acquire()
    eng.step([entry(sa, a[:79], [])])
    got = eng.step([entry(sa, a[79:], [0]), entry(sb, b, range(37))])
    close(got[:1], P.forward(cfg, w, a)[-1:], "float32")
    close(got[1:], P.forward(cfg, w, b), "float32")
    eng.release(sa)
    eng.release(sb)


@pytest.mark.parametrize("name", list(MODELS))
def test_greedy_generation_through_the_library(folders, plain, name):
    import hector_engine_amd as he
    cfg, w = plain[name]
    prompts = [rand_ids(cfg["vocab"], n, 70 + i) for i, n in enumerate([5, 30, 61])]
    steps = 40
    want = [P.greedy(cfg, w, p, steps) for p in prompts]
    eng = he.Engine(folders[name], dtype="float32", max_tokens=2048, max_seq_len=512)
    got = he.generate(eng, prompts, max_new_tokens=steps, stop_ids=())
    assert [r.tokens for r in got] == want
    small = he.Engine(folders[name], dtype="float32", max_tokens=2048, max_slots=2, max_seq_len=512)
    assert [r.tokens for r in he.generate(small, prompts, max_new_tokens=steps, stop_ids=())] == want
    assert small.cache.free_pages == small.cache.num_pages
    eng16 = he.Engine(folders[name], dtype="bfloat16", max_tokens=2048, max_seq_len=512)
    for p, r, t in zip(prompts, he.generate(eng16, prompts, max_new_tokens=steps, stop_ids=()), want):
        seq = list(p)
        for x, y in zip(r.tokens, t):
            if x != y:
                top = P.forward(cfg, w, seq)[-1].topk(2).values
                assert (top[0] - top[1]).item() < 0.03 * top[0].abs().item() + 1e-3      # a near tie
                break
            seq.append(x)


def test_the_command_line_and_the_trace_replay_serve_it(folders, plain, tmp_path):
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    from tests.conftest import ROOT
    cfg, w = plain["V1"]
    exe = os.path.join(ROOT, "bin", "hector_generate")
    out = subprocess.run([sys.executable, exe, folders["V1"], "5,17,3;9,2,77,13", "6", "--dtype", "float32",
                          "--stop-ids", ""], capture_output=True, text=True, timeout=180)
    assert out.returncode == 0, out.stderr
    for i, p in enumerate(([5, 17, 3], [9, 2, 77, 13])):
        assert f"[{i}] prompt" in out.stdout and ",".join(map(str, P.greedy(cfg, w, p, 6))) in out.stdout
    assert "Volonex" in out.stdout
    # a replay whose requests need more pages than their token count alone suggests (each request's
    # last page is partly empty): 196 tokens live at once, in 1 + 2 + 3 pages
    reqs = {"a": rand_ids(cfg["vocab"], 4, 1), "b": rand_ids(cfg["vocab"], 68, 2), "c": rand_ids(cfg["vocab"], 133, 3)}
    steps = [{"step": 0, "entries": [{"id": k, "tokens": v[:-3], "want": [len(v) - 4]} for k, v in reqs.items()], "end": []}]
    for t in range(3):
        steps.append({"step": t + 1, "entries": [{"id": k, "tokens": [v[len(v) - 3 + t]], "want": [0]} for k, v in reqs.items()],
                      "end": list(reqs) if t == 2 else []})
    for dtype in DTYPES:
        out_dir = str(tmp_path / dtype)
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders["V1"],
                               "--dtype", dtype, "--out", out_dir, "--max-tokens", "196"],
                              input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=180)
        assert proc.returncode == 0, proc.stderr
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
        want = {k: P.forward(cfg, w, v) for k, v in reqs.items()}
        for s in range(4):
            got = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{s}.f32"), dtype="<f4").reshape(3, -1).copy())
            rows = torch.stack([want[k][len(reqs[k]) - 4 + s] for k in reqs])
            close(got, rows, dtype)


def test_pages_before_the_running_chunk_go_back_to_the_pool(engines, plain):
    eng = engines("V2", "float32")
    cfg, w = plain["V2"]
    ids = rand_ids(cfg["vocab"], 300, 5)
    free = eng.cache.free_pages
    s = eng.acquire()
    eng.step([entry(s, ids[:290], [])])
    got = torch.cat([eng.step([entry(s, [t], [0])]).clone() for t in ids[290:]])
    close(got, P.forward(cfg, w, ids)[290:], "float32")
    held = {g.chunk: sum(p >= 0 for p in g.table[s]) for g in eng.cache.book.groups}
    assert held == {16: 1, 0: 5, 128: 1}          # 300 tokens lie in five pages; the chunks that run began at 288 and 256
    eng.release(s)
    assert eng.cache.free_pages == free
