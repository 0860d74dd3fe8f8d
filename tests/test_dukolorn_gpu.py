"""The Dukolorn decoder on the GPU against the plain implementation (tests/plain/dukolorn.py):
every mechanism's kernels alone and as parts over portions and single tokens, keys made to stand
out (far back, at page borders, just inside and just outside a window), the sink and the bias by
distance shown by weights that make them decide, whole models of three tiny configurations under
the four schedule families in float32 and bfloat16 with pools so small that pages and slots are
used again, long decoding, a batch against its requests alone, and greedy generation through the
engine and its scheduler."""
import math

import numpy as np
import pytest
import torch

import emulated_ops as E
import schedules
from plain import dukolorn as P
from replay_common import collect, make_requests
from tiny_dukolorn import TINY, assert_matches_plain, read_model_dir, write_tiny

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16, F64 = torch.float32, torch.bfloat16, torch.float64


def gen(seed):
    return torch.Generator().manual_seed(seed)


def rel(got, want):
    got = got.detach().to("cpu", F64)
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def dev_i32(a):
    return torch.tensor(a, dtype=torch.int32, device=DEV)


def tables(segments, slots=None):
    """int32 row tables for segments [(first position, rows), ...]: on the GPU and on the host."""
    row_pos, row_seg, seg_start = [], [], [0]
    for s, (p0, n) in enumerate(segments):
        row_pos += list(range(p0, p0 + n))
        row_seg += [s] * n
        seg_start.append(seg_start[-1] + n)
    slots = list(range(len(segments))) if slots is None else slots
    host = dict(row_pos=row_pos, row_seg=row_seg, seg_start=seg_start,
                seg_pos0=[p for p, _ in segments], seg_slot=slots)
    host = {k: torch.tensor(v, dtype=torch.int32) for k, v in host.items()}
    return {k: v.to(DEV) for k, v in host.items()}, host


def bind_random(part, seed, dtype, std=0.2, change=None):
    from kappai_amd.weights import random_tensors, stored_to_runtime
    t = random_tensors(part.tensor_specs(), seed, std=std)
    if change:
        change(t)
    part.bind({k: stored_to_runtime(v, dtype).to(DEV) for k, v in t.items()})
    return t


def step_through(part, cm, x, portions, view):
    """One request through a mixer in ``portions``; returns the outputs in order."""
    from test_parts_gpu import one_segment_batch
    rc, outs, done = None, [], 0
    for n in portions:
        rc, b = one_segment_batch(cm, n, rc=rc)
        y = part.forward(x[done:done + n].to(DEV), b, view)
        outs.append(y if y.dim() == 2 else y.sum(0))
        cm.commit(rc, n)
        cm.check()
        done += n
    assert done == x.shape[0]
    return torch.cat(outs).float(), rc


PORTIONS_150 = [37, 3] + [1] * 50 + [2, 33] + [1] * 25


# ---------------------------------------------------------------------------------------------
# kernels alone
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("D", [72, 64, 328, 2048, 100])
def test_norm_on_a_sublayers_output(D):
    from kappai_amd.kernels import ops
    T = 19
    x = torch.randn(T, D, generator=gen(1)) * 3
    w = 1 + 0.2 * torch.randn(D, generator=gen(2))
    for kind in ("f32", "bf16", "parts", "two", "set"):
        a = torch.randn(T, D, generator=gen(3))
        b = None
        if kind == "bf16":
            a = a.to(BF16)
        elif kind == "parts":
            a = torch.randn(5, T, D, generator=gen(4))
        elif kind == "two":
            a, b = a.to(BF16), torch.randn(T, D, generator=gen(5)).to(BF16)
        y = (a.double().sum(0) if a.dim() == 3 else a.double()) * 0.7
        if b is not None:
            y = y + 1.3 * b.double()
        n = P.norm_plain(y, w, 1e-5)
        want = n if kind == "set" else x.double() + n
        resid = x.clone().to(DEV)
        rows = ops.output_norm_add(resid, a.to(DEV), w.to(DEV), 1e-5, rows_dtype=BF16, scale_a=0.7,
                                   b=None if b is None else b.to(DEV), scale_b=1.3,
                                   add=kind != "set")
        assert rel(resid, want) < 2e-6, kind
        assert torch.equal(rows.cpu(), resid.cpu().to(BF16))


@pytest.mark.parametrize("taps", [1, 2, 4, 5])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_convolution_with_silu_over_portions_and_slots(taps, dtype):
    """Two requests side by side in slots 3 and 1 of states that hold NaN, in portions down to one
    row, against the whole sequences at once."""
    from kappai_amd.kernels import ops
    C, T = 40, 31
    w = torch.randn(C, taps, generator=gen(6)) * 0.5
    xs = [torch.randn(T, C + 8, generator=gen(7 + i)).to(BF16) for i in range(2)]
    state = torch.full((5, taps - 1, C), float("nan"), device=DEV)
    outs, done = [[], []], 0
    for n in [5, 1, 1, 2, 9, 1, 12]:
        tb, _ = tables([(done, n), (done, n)], slots=[3, 1])
        x = torch.cat([xs[0][done:done + n], xs[1][done:done + n]]).to(dtype).to(DEV)
        y = ops.conv_silu(x, w.to(DEV), state, tb["row_pos"], tb["row_seg"], tb["seg_start"],
                          tb["seg_pos0"], tb["seg_slot"])
        outs[0].append(y[:n])
        outs[1].append(y[n:])
        done += n
    for i in range(2):
        want = P.conv_silu(xs[i][:, :C].double(), w)
        assert rel(torch.cat(outs[i]).float(), want) < (1e-5 if dtype == F32 else 1e-2)


@pytest.mark.parametrize("H,Hk,d,dv,delta", [(3, 3, 8, 16, False), (4, 2, 8, 16, True),
                                             (1, 1, 72, 24, False), (2, 2, 136, 8, True),
                                             (2, 1, 24, 70, True), (1, 1, 40, 8, False),
                                             (2, 2, 128, 128, True), (2, 1, 64, 136, False),
                                             (1, 1, 300, 4, True), (1, 1, 16, 600, True),
                                             (2, 2, 260, 40, False), (3, 1, 10, 6, True)])
@pytest.mark.parametrize("form", ["wave", "block", "auto"])
def test_matrix_state_recurrence_against_the_stand_in(H, Hk, d, dv, delta, form):
    """Both recurrences over three requests in portions (slots used in another order, NaN in the
    states before), against the torch stand-in of the same operation run on whole sequences; by
    the kernel that reads token by token and by the one that takes chunks through LDS (portions of
    20 and 13 tokens end inside a chunk)."""
    from kappai_amd.kernels import ops
    if form == "block" and d % 4:
        pytest.skip("the kernel that works through LDS takes key sizes that are multiples of four")
    T = 45
    g = gen(8)
    seqs = []
    for _ in range(3):
        seqs.append(dict(q=torch.randn(T, Hk * d, generator=g), k=torch.randn(T, Hk * d, generator=g),
                         v=torch.randn(T, H * dv, generator=g), z=torch.randn(T, H * d, generator=g) * 2,
                         b=torch.randn(T, H, generator=g)))
    rate = torch.rand(H, generator=g) + 0.1
    zb = torch.randn(H * d, generator=g)
    kw = dict(unit_qk=delta, unit_eps=1e-6)
    sign = 1.0 if delta else -1.0
    want = []
    for s in seqs:
        st = torch.zeros(1, H, dv, d)
        tb = {k: torch.tensor(v, dtype=torch.int32) for k, v in
              dict(seg_start=[0, T], seg_pos0=[0], seg_slot=[0]).items()}
        want.append(E.matrix_state_recurrence(s["q"], s["k"], s["v"], s["z"], H, Hk, d, dv, rate,
                                              zb, sign, d ** -0.5, st, tb["seg_start"],
                                              tb["seg_pos0"], tb["seg_slot"],
                                              beta=s["b"] if delta else None, **kw))
    state = torch.full((6, H, dv, d), float("nan"), device=DEV)
    got, done = [[], [], []], 0
    for n in [7, 1, 2, 1, 20, 1, 13]:
        tb, _ = tables([(done, n)] * 3, slots=[4, 0, 2])
        cat = {k: torch.cat([s[k][done:done + n] for s in seqs]).to(DEV) for k in "qkvzb"}
        o = ops.matrix_state_recurrence(cat["q"], cat["k"], cat["v"], cat["z"], H, Hk, d, dv,
                                        rate.to(DEV), zb.to(DEV), sign, d ** -0.5, state,
                                        tb["seg_start"], tb["seg_pos0"], tb["seg_slot"],
                                        beta=cat["b"] if delta else None, form=form, **kw)
        for i in range(3):
            got[i].append(o[i * n:(i + 1) * n])
        done += n
    for i in range(3):
        assert rel(torch.cat(got[i]), want[i].double()) < 2e-5, i


@pytest.mark.parametrize("H,n_in,n_out,T,pad", [(3, 16, 20, 37, 4), (1, 40, 8, 1, 4),
                                                (4, 8, 100, 70, 4), (2, 33, 65, 5, 4),
                                                (3, 16, 20, 37, 8), (1, 40, 8, 1, 0),
                                                (4, 72, 100, 70, 16), (2, 192, 130, 16, 64),
                                                (5, 24, 64, 17, 8), (2, 128, 192, 200, 0)])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_a_matrix_per_head(H, n_in, n_out, T, pad, dtype):
    """Heads that stand ``n_in + pad`` apart in rows of a few values more; in bfloat16 the paddings
    that keep every head at a multiple of eight values run on the matrix cores, the others and
    float32 on the plain kernel."""
    from kappai_amd.kernels import ops
    step = n_in + pad
    x = torch.randn(T, H * step + 8, generator=gen(9)).to(BF16)
    w = (torch.randn(H, n_out, n_in, generator=gen(10)) * 0.3).to(BF16)
    out = torch.zeros(T, H * (n_out + 2), dtype=dtype, device=DEV)
    ops.headwise_linear(x.to(dtype).to(DEV), step, w.to(dtype).to(DEV), out=out,
                        out_head_stride=n_out + 2)
    for h in range(H):
        want = x[:, h * step:h * step + n_in].double() @ w[h].double().T
        got = out[:, h * (n_out + 2):h * (n_out + 2) + n_out]
        assert rel(got.float(), want) < (1e-5 if dtype == F32 else 1e-2)
        assert float(out[:, h * (n_out + 2) + n_out:(h + 1) * (n_out + 2)].abs().max()) == 0.0


@pytest.mark.parametrize("kernel", ["rows", "prefill", "decode-block", "decode-split"])
@pytest.mark.parametrize("H,G,D,window,n_keys", [(6, 2, 32, 0, 150), (4, 4, 16, 37, 300),
                                                 (3, 1, 64, 0, 700), (8, 2, 128, 72, 90),
                                                 (5, 1, 96, 50, 200), (16, 1, 192, 0, 300),
                                                 (4, 2, 48, 0, 130), (2, 1, 256, 64, 150)])
@pytest.mark.parametrize("what", ["all", "sink"])
def test_attention_kernels_work_on_the_scores(kernel, H, G, D, window, n_keys, what):
    """Cap, bias by distance and sink (or the sink alone, which leaves the scores to the kernels'
    plain path) in every attention kernel (bfloat16; the plain kernel also in float32), one
    request of ``n_keys`` keys and a second short one, against the stand-in.  The bias table ends
    40 keys back: most key tiles of the long request lie beyond it."""
    from kappai_amd.kernels import ops
    ps = 16
    lens = [n_keys, 21]
    g = gen(11)
    pages = sum((n + ps - 1) // ps for n in lens)
    k_pool = (torch.randn(pages + 1, G, ps, D, generator=g)).to(BF16)
    v_pool = (torch.randn(pages + 1, G, D, ps, generator=g)).to(BF16)
    order = torch.randperm(pages, generator=g).tolist()
    bt = torch.full((2, (n_keys + ps - 1) // ps), -1, dtype=torch.int32)
    at = 0
    for s, n in enumerate(lens):
        for b in range((n + ps - 1) // ps):
            bt[s, b] = order[at]
            at += 1
    mods_host = ops.ScoreMods(2.5, torch.randn(H, 40, generator=g), torch.randn(H, generator=g) + 2)
    if what == "sink":
        mods_host = ops.ScoreMods(0.0, None, mods_host.sink)
    mods = ops.ScoreMods(mods_host.softcap,
                         None if what == "sink" else mods_host.distance_bias.to(DEV),
                         mods_host.sink.to(DEV))
    if kernel in ("decode-block", "decode-split"):
        segs = [(lens[0] - 1, 1), (lens[1] - 1, 1)]
    else:
        segs = [(lens[0] - 40, 40), (lens[1] - 9, 9)]
    tb, host = tables(segs)
    T = int(host["row_pos"].shape[0])
    q = (torch.randn(T, H * D, generator=g) * 0.5).to(BF16)
    tiles = []
    for s, (p0, n) in enumerate(segs):
        for j in range(0, n, 32):
            tiles.append([s, int(host["seg_start"][s]) + j, min(32, n - j), 0])
    want = E.paged_attention(q.float(), H, G, D, k_pool.float(), v_pool.float(), host["row_pos"],
                             host["row_seg"], bt, ps, 0.3, window=window, mods=mods_host).double()
    dtypes = [BF16, F32] if kernel == "rows" else [BF16]
    for dtype in dtypes:
        got = ops.paged_attention(
            q.to(dtype).to(DEV), H, G, D, k_pool.to(dtype).to(DEV), v_pool.to(dtype).to(DEV),
            tb["row_pos"], tb["row_seg"], bt.to(DEV), ps, 0.3, window=window,
            q_tiles=dev_i32(tiles), single_rows=kernel.startswith("decode"),
            max_position=max(lens) - 1, kernel=kernel, mods=mods)
        assert rel(got.float(), want) < (2e-2 if dtype == BF16 else 1e-5), dtype
    # the sink alone changes the result (it is not dropped somewhere on the way)
    bare = E.paged_attention(q.float(), H, G, D, k_pool.float(), v_pool.float(), host["row_pos"],
                             host["row_seg"], bt, ps, 0.3, window=window,
                             mods=ops.ScoreMods(mods_host.softcap, mods_host.distance_bias,
                                                None)).double()
    assert float((bare - want).abs().max()) > 0.05


# ---------------------------------------------------------------------------------------------
# the mixers as parts, over portions and single tokens
# ---------------------------------------------------------------------------------------------
def scored_part(dtype, H, G, d, dv, window=None, **kw):
    from kappai_amd.parts import ScoredAttention
    opts = dict(norm_eps=1e-5, whole_qk_norm=True, softcap=6.0, bias_buckets=10, bias_far=45.0,
                sink=True, temp_coef=0.4, temp_every=16, weight_suffix="")
    opts.update(kw)
    return ScoredAttention("a.", 72, H, G, d, dv, 0.25, dtype, window=window, **opts)


def scored_dict(H, G, d, dv, **kw):
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": 0.25, "softcap": 6.0,
         "bias_max": 45.0, "q_temp": {"coef": 0.4, "every": 16}}
    m.update(kw)
    return m


@pytest.mark.parametrize("dtype,tol", [(F32, 2e-5), (BF16, 3e-2)])
@pytest.mark.parametrize("H,G,d,dv", [(6, 2, 16, 24), (3, 3, 24, 16), (1, 1, 40, 8), (8, 1, 16, 16),
                                      (18, 1, 16, 16), (40, 2, 8, 16)])
def test_scored_attention_part(dtype, tol, H, G, d, dv):
    from kappai_amd.cache import CacheManager
    part = scored_part(dtype, H, G, d, dv)
    t = bind_random(part, 3, dtype)
    cm = CacheManager([part.cache_spec()], 16, 12, 1)
    cm.allocate_storage(dtype, DEV, poison=True)
    x = torch.randn(150, 72, generator=gen(14)).to(BF16)
    got, _ = step_through(part, cm, x.to(dtype), PORTIONS_150, cm.view(0))
    want = P.biased_attention(x.double(), t, "a.", scored_dict(H, G, d, dv), 1e-5)
    assert rel(got, want) < tol


def needle_rows(T, needle, half, seed):
    """[T, 2 half] rows whose first half is what queries read and whose second half is what keys
    read.  Every query after the needle points along ``u``; the needle's key does too, every other
    key lies along ``r`` (at right angles to ``u``) but for a little noise: all of a later query's
    weight falls on the needle, wherever it is."""
    u = torch.ones(half) / math.sqrt(half)
    r = u * torch.tensor([1.0, -1.0]).repeat(half // 2)
    x = torch.randn(T, 2 * half, generator=gen(seed)) * 0.02
    x[:, half:] += r
    x[needle, half:] = 3.0 * u
    x[needle + 1:, :half] += 1.5 * u
    return x.to(BF16)


@pytest.mark.parametrize("dtype,tol", [(F32, 1e-4), (BF16, 5e-2)])
def test_scored_attention_finds_a_far_key_and_weighs_bias_and_sink(dtype, tol):
    """Queries read the first half of the input and keys the second (identity maps; the norm over
    the whole projection gives every key the same length, so only its direction counts): one needle
    row gets all the weight of every later query, at position 0, at page borders and 400 keys
    back, in a portion and token by token.  Then the same with a bias table that shuts out
    everything further than its linear half (the needle is lost), and with a sink so large that
    nothing else counts."""
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import ScoredAttention
    H = G = 2
    d = dv = 16
    half = H * d
    W = 2 * half

    def build(rel_far=0.0, sink=-20.0):
        part = ScoredAttention("a.", W, H, G, d, dv, 1.0, dtype, norm_eps=1e-5, whole_qk_norm=True,
                               softcap=40.0, bias_buckets=8, bias_far=20.0, sink=True,
                               weight_suffix="")

        def change(t):
            eye, zero = torch.eye(half), torch.zeros(half, half)
            t["a.q"] = torch.cat([eye, zero], 1).to(BF16)
            t["a.k"] = torch.cat([zero, eye], 1).to(BF16)
            t["a.q.norm"] = torch.full((half,), 4.0).to(BF16)
            t["a.k.norm"] = torch.full((half,), 1.0).to(BF16)
            rel_t = torch.zeros(8, H)
            rel_t[4:] = rel_far
            t["a.rel"] = rel_t.to(BF16)
            t["a.sink"] = torch.full((H,), sink).to(BF16)
        return part, bind_random(part, 4, dtype, std=0.3, change=change)

    m = scored_dict(H, G, d, dv, scale=1.0, softcap=40.0, bias_max=20.0,
                    q_temp={"coef": 0.0, "every": 1})
    for needle in (0, 15, 16, 63):
        T = needle + 403
        x = needle_rows(T, needle, half, needle)
        for rel_far, sink in ((0.0, -20.0), (-60.0, -20.0), (0.0, 60.0)):
            part, t = build(rel_far, sink)
            want = P.biased_attention(x.double(), t, "a.", m, 1e-5)
            for portions in ([needle + 1, T - needle - 7] + [1] * 6, [needle + 2, T - needle - 2]):
                cm = CacheManager([part.cache_spec()], 16, T // 16 + 2, 1)
                cm.allocate_storage(dtype, DEV, poison=True)
                got, _ = step_through(part, cm, x.to(dtype), portions, cm.view(0))
                err = (got.cpu().double() - want).abs().max(dim=1).values / want.abs().max()
                assert float(err.max()) < tol, (needle, rel_far, sink, int(err.argmax()))
        # what the three cases must look like: found; lost beyond the table's half; drowned
        part, t = build()
        found = P.biased_attention(x.double(), t, "a.", m, 1e-5)[-1]
        lost = P.biased_attention(x.double(), build(-60.0)[1], "a.", m, 1e-5)[-1]
        drowned = P.biased_attention(x.double(), build(0.0, 60.0)[1], "a.", m, 1e-5)[-1]
        assert float((found - lost).abs().max()) > 0.2 * float(found.abs().max())
        assert float(drowned.abs().max()) < 1e-3 * float(found.abs().max())


@pytest.mark.parametrize("dtype,tol", [(F32, 2e-5), (BF16, 3e-2)])
@pytest.mark.parametrize("H,d,rot,dv,r,dims,window", [(3, 16, 8, 24, 20, 8, 21),
                                                      (2, 8, 16, 8, 40, 12, None),
                                                      (4, 8, 8, 16, 24, 8, 1),
                                                      (2, 24, 8, 8, 16, 8, 33),
                                                      (20, 8, 8, 8, 16, 8, 21),
                                                      (17, 16, 16, 8, 64, 16, None)])
def test_latent_attention_part(dtype, tol, H, d, rot, dv, r, dims, window):
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import LatentAttention, RotaryEncoding
    part = LatentAttention("a.", 72, H, d, rot, dv, r, 0.2, 1e-5, dtype,
                           position=RotaryEncoding(rot, 700.0, rot_dim=dims, pairing="interleaved"),
                           window=window, sink=True, weight_suffix="")
    t = bind_random(part, 5, dtype)
    cm = CacheManager([part.cache_spec()], 16, 12, 1)
    cm.allocate_storage(dtype, DEV, poison=True)
    x = torch.randn(150, 72, generator=gen(15)).to(BF16)
    got, rc = step_through(part, cm, x.to(dtype), PORTIONS_150, cm.view(0))
    m = {"heads": H, "dim": d, "rot_dim": rot, "vdim": dv, "kv_rank": r, "scale": 0.2,
         "rot": {"base": 700.0, "dims": dims}}
    if window is not None:
        m["mask"] = {"size": window}
        assert rc.blocks[0][0] == -1           # pages the window has passed went back
    assert rel(got, P.latent_attention(x.double(), t, "a.", m, 1e-5)) < tol


@pytest.mark.parametrize("dtype,tol", [(F32, 1e-4), (BF16, 5e-2)])
@pytest.mark.parametrize("window", [70, 200])
def test_latent_attention_sees_a_key_just_inside_its_window_and_not_just_outside(dtype, tol,
                                                                                 window):
    """The latent is the input itself (an identity map, norm weight of one), keys and queries read
    it through identity up-projections, nothing rotates: one needle row gets all the weight of
    every later query while the window holds it and none one position later."""
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import LatentAttention
    H, d, r = 2, 16, 32
    W = 2 * r
    part = LatentAttention("a.", W, H, d, 0, d, r, 1.0, 1e-5, dtype, position=None, window=window,
                           sink=True, weight_suffix="")

    def change(t):
        eye, zero = torch.eye(r), torch.zeros(r, r)
        t["a.q"] = torch.cat([eye, zero], 1).to(BF16)
        t["a.dkv"] = torch.cat([zero, eye], 1).to(BF16)
        t["a.dkv.norm"] = torch.full((r,), 1.0).to(BF16)
        t["a.uk"] = (torch.eye(r) * 6.0).to(BF16)
        t["a.sink"] = torch.full((H,), -5.0).to(BF16)
    t = bind_random(part, 6, dtype, std=0.3, change=change)
    m = {"heads": H, "dim": d, "rot_dim": 0, "vdim": d, "kv_rank": r, "scale": 1.0,
         "rot": {"base": 10.0, "dims": 0}, "mask": {"size": window}}
    for needle in (0, 15, 16, 63, 100):
        T = needle + window + 3
        x = needle_rows(T, needle, r, needle)
        want = P.latent_attention(x.double(), t, "a.", m, 1e-5)
        inside, outside = want[needle + window - 1], want[needle + window]
        assert float((inside - outside).abs().max() / want.abs().max()) > 0.2
        for portions in ([needle + 1, T - needle - 7] + [1] * 6, [needle + 2, T - needle - 2]):
            cm = CacheManager([part.cache_spec()], 16, T // 16 + 2, 1)
            cm.allocate_storage(dtype, DEV, poison=True)
            got, _ = step_through(part, cm, x.to(dtype), portions, cm.view(0))
            err = (got.cpu().double() - want).abs().max(dim=1).values / want.abs().max()
            assert float(err.max()) < tol, (needle, int(err.argmax()), float(err.max()))


@pytest.mark.parametrize("dtype,tol", [(F32, 3e-5), (BF16, 4e-2)])
@pytest.mark.parametrize("H,d,dv,tau,rank", [(3, 8, 16, 6.0, 5), (1, 72, 24, 3.0, 8),
                                             (2, 40, 8, 1.0, 4)])
def test_gated_linear_attention_part(dtype, tol, H, d, dv, tau, rank):
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import GatedLinearAttention
    part = GatedLinearAttention("a.", 72, H, d, dv, tau, rank, 1e-5, dtype, weight_suffix="",
                                bias_suffix=".b")
    t = bind_random(part, 7, dtype)
    cm = CacheManager([part.cache_spec()], 16, 1, 2)
    cm.allocate_storage(dtype, DEV, poison=True)
    x = torch.randn(150, 72, generator=gen(16)).to(BF16)
    got, _ = step_through(part, cm, x.to(dtype), PORTIONS_150, cm.view(0))
    m = {"heads": H, "dim": d, "vdim": dv, "tau": tau}
    assert rel(got, P.gated_linear_attention(x.double(), t, "a.", m, 1e-5)) < tol


@pytest.mark.parametrize("dtype,tol", [(F32, 3e-5), (BF16, 4e-2)])
@pytest.mark.parametrize("H,G,d,dv,taps", [(4, 2, 8, 16, 3), (1, 1, 24, 8, 1), (2, 2, 136, 8, 5),
                                           (6, 2, 16, 40, 4)])
def test_delta_rule_part(dtype, tol, H, G, d, dv, taps):
    from kappai_amd.cache import CacheManager
    from kappai_amd.parts import GatedDeltaRule
    part = GatedDeltaRule("a.", 72, H, G, d, dv, taps, 6, 7, 1e-5, dtype, weight_suffix="")
    t = bind_random(part, 8, dtype)
    cm = CacheManager([part.cache_spec()], 16, 1, 2)
    cm.allocate_storage(dtype, DEV, poison=True)
    x = torch.randn(150, 72, generator=gen(17)).to(BF16)
    got, _ = step_through(part, cm, x.to(dtype), PORTIONS_150, cm.view(0))
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "conv": taps}
    assert rel(got, P.channel_delta(x.double(), t, "a.", m, 1e-5)) < tol


def test_delta_rule_overwrites_what_a_key_held():
    """With beta near one and no decay, writing a second value under the same unit key replaces the
    first: a read with that key returns the second value alone (a plain sum would return both)."""
    from kappai_amd.kernels import ops
    d, dv = 8, 4
    k = torch.zeros(3, d)
    k[:, 2] = 5.0
    v = torch.tensor([[1.0, 2.0, 3.0, 4.0], [-4.0, 0.5, 9.0, 2.0], [0.0, 0.0, 0.0, 0.0]])
    z = torch.full((3, d), -40.0)                   # softplus(-40) = 0: the decay is one
    beta = torch.tensor([[40.0], [40.0], [-40.0]])    # write, overwrite, read only
    tb, _ = tables([(0, 3)])
    state = torch.full((1, 1, dv, d), float("nan"), device=DEV)
    o = ops.matrix_state_recurrence(k.to(DEV), k.to(DEV), v.to(DEV), z.to(DEV), 1, 1, d, dv,
                                    torch.ones(1, device=DEV), None, 1.0, 1.0, state,
                                    tb["seg_start"], tb["seg_pos0"], tb["seg_slot"],
                                    beta=beta.to(DEV), unit_qk=True)
    assert rel(o[2], v[1].double()) < 1e-5 and rel(o[0], v[0].double()) < 1e-5


# ---------------------------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------------------------
LENGTHS = {"U": [70, 45, 100, 37], "V": [66, 35, 90], "W": [50, 81, 36], "X": [130, 60, 90]}
MIXED_LENGTHS = {"U": [70, 45, 100, 37, 83, 64, 29, 58], "V": [66, 35, 90, 41, 23, 77, 50, 62, 88],
                 "W": [50, 81, 36, 67, 44, 72, 90, 33, 58], "X": [130, 60, 90, 41, 75, 100, 33]}


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("dukolorn")
    return {name: write_tiny(name, base / name) for name in TINY}


_models = {}


def gpu_model(model_dir, dtype):
    from kappai_amd.models import load_model
    key = (str(model_dir), dtype)
    if key not in _models:
        _models[key] = load_model(model_dir, dtype, DEV)
    return _models[key]


def replay(model_dir, dtype, steps, index, max_tokens, out_dir, slots=4, graphs=True):
    from kappai_amd.engine.replay import TraceReplayer, make_replay_cache
    from kappai_amd.engine.step import StepRunner
    model = gpu_model(model_dir, dtype)
    cache = make_replay_cache(model, max_tokens, 16, num_slots=slots)
    cache.allocate_storage(model.dtype, DEV, poison=True)
    runner = StepRunner(model, cache, DEV, decode_graphs=graphs)
    rep = TraceReplayer(runner, out_dir)
    outputs = {}
    for obj in steps:
        res = rep.run_step(obj)
        if res is not None:
            outputs[obj["step"]] = res
    cache.check()
    assert not cache.live_requests()
    return collect(index, outputs, model.vocab_size), runner


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["U", "V", "W", "X"])
@pytest.mark.parametrize("family", ["whole", "prefill_then_decode", "changing_portions", "mixed"])
def test_schedules(tmp_path, model_dirs, name, family, dtype):
    """Every logit of every request.  The mixed family runs in a pool smaller than its requests
    together with four state slots, so pages and slots are taken again."""
    requests = make_requests(TINY[name][0]["vocab"],
                             MIXED_LENGTHS[name] if family == "mixed" else LENGTHS[name], seed=21)
    steps, index, peak = getattr(schedules, family)(requests)
    if family == "mixed":
        assert sum(len(t) for t in requests.values()) > peak
    got, runner = replay(model_dirs[name], dtype, steps, index, peak, tmp_path / "out")
    assert len(got) == sum(len(t) for t in requests.values())
    assert_matches_plain(got, model_dirs[name], requests, dtype, (name, family, dtype))
    if family == "prefill_then_decode":
        assert runner.graph_replays > 0        # single tokens ran from captured graphs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_every_window(tmp_path, model_dirs, dtype):
    """A short prompt and 330 tokens one by one (windows of 1, 21 and 33 passed many times, pages
    given back and taken again, the block tables of a graph grown, the temperature's steps and the
    bias table's end passed), two requests side by side."""
    for name in ("U", "W"):
        requests = make_requests(TINY[name][0]["vocab"], [350, 290], seed=22)
        plans = {"r0": (0, [20] + [1] * 330), "r1": (5, [3] + [1] * 287)}
        steps, index, peak = schedules.build(requests, plans)
        got, runner = replay(model_dirs[name], dtype, steps, index, peak, tmp_path / name)
        assert_matches_plain(got, model_dirs[name], requests, dtype, (name, dtype))
        assert runner.graph_replays > 250


def test_a_batch_gives_what_its_requests_give_alone(tmp_path, model_dirs):
    """Unequal requests in one step (a long portion, a short one, single tokens) against each
    request stepped alone: the same logits up to rounding, with and without graphs."""
    requests = make_requests(TINY["U"][0]["vocab"], [120, 9, 40], seed=23)
    alone, _ = replay(model_dirs["U"], "float32", *schedules.changing_portions(requests),
                      tmp_path / "alone", graphs=False)
    plans = {"r0": (0, [100] + [1] * 20), "r1": (1, [2, 2] + [1] * 5), "r2": (0, [1, 30, 2, 7])}
    together, _ = replay(model_dirs["U"], "float32", *schedules.build(requests, plans),
                         tmp_path / "together")
    assert alone.keys() == together.keys()
    scale = max(float(np.abs(v).max()) for v in alone.values())
    worst = max(float(np.abs(alone[k] - together[k]).max()) / scale for k in alone)
    assert worst < 1e-5


def test_the_residual_stream_layer_by_layer(model_dirs):
    """The stream after every layer of a whole prompt, in float32, against the plain
    implementation's."""
    from kappai_amd.cache import CacheManager
    from kappai_amd.engine import StepEntry, StepRunner
    name = "U"
    model = gpu_model(model_dirs[name], "float32")
    cfg, t = read_model_dir(model_dirs[name])
    tokens = [int(x) for x in np.random.default_rng(3).integers(0, cfg["vocab"], size=41)]
    streams = []
    P.forward(cfg, t, tokens, streams=streams)
    cm = CacheManager(model.cache_specs(), 16, 8, 1)
    cm.allocate_storage(model.dtype, DEV, poison=True)
    runner = StepRunner(model, cm, DEV, decode_graphs=False)
    seen = []
    for layer in model.layers:
        inner = layer.forward

        def spy(h, batch, cache, shared_cache=False, inner=inner):
            out = inner(h, batch, cache, shared_cache=shared_cache)
            seen.append(out.resid.detach().clone())
            return out
        layer.forward = spy
    try:
        runner.step([StepEntry(cm.open("a"), tokens, [len(tokens) - 1])])
    finally:
        for layer in model.layers:
            del layer.forward
    assert len(seen) == len(streams)
    for i, (got, want) in enumerate(zip(seen, streams)):
        assert rel(got, want) < 2e-5, i


def test_greedy_generation_through_the_engine(model_dirs):
    """Prompts of unequal length through ``Engine.generate`` (its scheduler cuts the prompts into
    portions of 16 beside decoding) against the plain implementation's greedy choice."""
    from kappai_amd.engine import Engine
    from kappai_amd.sampling import SamplingParams
    for name in ("U", "V"):
        rng = np.random.default_rng(5)
        prompts = [[int(t) for t in rng.integers(0, TINY[name][0]["vocab"], size=n)]
                   for n in (45, 7, 23)]
        cfg, t = read_model_dir(model_dirs[name])
        want = []
        for p in prompts:
            toks = list(p)
            for _ in range(10):
                toks.append(int(P.forward(cfg, t, toks)[-1].argmax()))
            want.append(toks[len(p):])
        eng = Engine(str(model_dirs[name]), dtype="float32", num_pages=24, max_batch=3, chunk=16,
                     token_budget=24)
        got = eng.generate(prompts, SamplingParams.greedy(n_predict=10))
        assert got == want
        assert eng.cache.num_free_slots == 3
        assert all(g.allocator.num_used == 0 for g in eng.cache.paged_groups)
        eng.shutdown()


def test_command_line(model_dirs, tmp_path):
    """The command line on a model folder and in random-weights mode (a named shape), with the
    sampling options of any other model; ``--time`` prints the stages of the new parts."""
    import subprocess
    import sys
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    prompt = [5, 17, 3, 88, 41, 7, 120]
    cfg, t = read_model_dir(model_dirs["U"])
    toks = list(prompt)
    for _ in range(6):
        toks.append(int(P.forward(cfg, t, toks)[-1].argmax()))
    out = subprocess.run(
        [sys.executable, "-m", "kappai_amd", "-m", str(model_dirs["U"]), "--dtype", "float32",
         "-p", ",".join(map(str, prompt)), "-n", "6", "-t", "0", "--num-pages", "16", "--time"],
        cwd=str(root), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert [int(x) for x in out.stdout.split()] == toks[len(prompt):]
    assert "scan" in out.stderr and "short_conv" in out.stderr and "attn" in out.stderr
    made = tmp_path / "made"
    out = subprocess.run(
        [sys.executable, str(root / "bin" / "kappai-cli"), "--random-weights", "dukolorn-tiny",
         "--model", str(made), "--weight-seed", "2", "--weight-std", "0.1", "-n", "5", "-t", "0.8",
         "-k", "20", "-s", "3", "--num-pages", "16", "7 8 9 10"],
        cwd=str(tmp_path), capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert len(out.stdout.split()) == 5 and (made / "config.json").is_file()
