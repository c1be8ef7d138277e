"""HIP kernels of the hybrid decoders (csrc/kernels/hybrid.hip) against the plain PyTorch fp32
versions of the same ops (ops/reference.py), one op at a time, in both activation types and at
sizes that are not multiples of anything convenient."""
import pytest
import torch

from llm_consensus_amd import ops
from llm_consensus_amd.ops import reference as ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ACTS = [torch.bfloat16, torch.float32]


def _tol(dt):
    return dict(atol=2e-2, rtol=2e-2) if dt == torch.bfloat16 else dict(atol=2e-5, rtol=2e-5)


def _seqs(lens, starts):
    """cu_q, positions, row_seq for sequences of the given lengths that start at the given positions."""
    cu, pos, rs = [0], [], []
    for b, (n, s) in enumerate(zip(lens, starts)):
        cu.append(cu[-1] + n)
        pos += list(range(s, s + n))
        rs += [b] * n
    i32 = lambda a: torch.tensor(a, dtype=torch.int32)  # noqa: E731
    return i32(cu), i32(pos), i32(rs)


@pytest.mark.parametrize("a_dt,w_dt,out_f32", [(torch.bfloat16, torch.bfloat16, True), (torch.float32, torch.bfloat16, True),
                                              (torch.float32, torch.float32, True), (torch.bfloat16, torch.bfloat16, False)])
@pytest.mark.parametrize("M,N,K", [(1, 7, 16), (5, 130, 100), (131, 64, 320), (70, 333, 48)])
def test_gemm_any(a_dt, w_dt, out_f32, M, N, K):
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    x = torch.randn(M, K, generator=g).to(a_dt)
    W = (torch.randn(N, K, generator=g) / K ** 0.5).to(w_dt)
    b = torch.randn(N, generator=g).to(w_dt)
    for relu2 in (False, True):
        w = ops.LinearWeight.from_dense(W, b, DEV, dtype=w_dt, any_shape=True)
        if w.is_packed:
            continue
        y = ops.linear_any(x.to(DEV), w, out_f32=out_f32, epi_relu2=relu2).float().cpu()
        want = x.float() @ W.float().T + b.float()
        want = torch.relu(want) ** 2 if relu2 else want
        tol = dict(atol=1e-4, rtol=1e-4) if out_f32 else dict(atol=3e-2, rtol=2e-2)
        torch.testing.assert_close(y, want, **tol)


@pytest.mark.parametrize("dt", ACTS)
def test_embed_rows_and_scalar_norm(dt):
    g = torch.Generator().manual_seed(1)
    E = torch.randn(50, 72, generator=g).to(dt)
    ids = torch.randint(0, 50, (9,), generator=g, dtype=torch.int32)
    x, xa = ops.embed_rows(ids.to(DEV), E.to(DEV), dt)
    torch.testing.assert_close(x.cpu(), E[ids.long()].float())
    torch.testing.assert_close(xa.float().cpu(), E[ids.long()].float())
    y = torch.randn(9, 72, generator=g)
    gain = torch.tensor([1.3])
    x0 = x.cpu().clone()
    want_a = ref.scalar_norm_add(x0, y, gain, 1e-5, dt)
    got_a = ops.scalar_norm_add(x, y.to(DEV), gain.to(DEV), 1e-5, dt)
    torch.testing.assert_close(x.cpu(), x0, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(got_a.float().cpu(), want_a.float(), **_tol(dt))
    fin = ops.scalar_norm_add(x, None, gain.to(DEV), 1e-5, dt)
    torch.testing.assert_close(fin.float().cpu(), ref.scalar_norm_add(x0, None, gain, 1e-5, dt).float(), **_tol(dt))
    torch.testing.assert_close(x.cpu(), x0, atol=1e-5, rtol=1e-5)          # untouched without an addend
    torch.testing.assert_close(ops.relu2(y.to(DEV), dt).float().cpu(), ref.relu2(y, dt).float(), **_tol(dt))
    rows = torch.tensor([3, 0, 8], dtype=torch.int32)
    torch.testing.assert_close(ops.gather_rows(x, rows.to(DEV)).cpu(), x0[rows.long()])


@pytest.mark.parametrize("dt", ACTS)
@pytest.mark.parametrize("w", [5, 130])
def test_mingru_scan(dt, w):
    g = torch.Generator().manual_seed(w)
    cu, pos, _ = _seqs([7, 1, 3, 1], [0, 9, 4, 0])
    slots = torch.tensor([2, 0, -1, 3], dtype=torch.int32)
    zxg = torch.randn(12, 3 * w, generator=g) * 2
    st = torch.randn(5, w, generator=g)
    st_ref = st.clone()
    want = ref.mingru_scan(zxg, st_ref, cu, pos, slots, dt)
    st_dev = st.to(DEV)
    got = ops.mingru_scan(zxg.to(DEV), st_dev, cu.to(DEV), pos.to(DEV), slots.to(DEV), dt)
    live = torch.tensor([True] * 8 + [False] * 3 + [True])
    torch.testing.assert_close(got.float().cpu()[live], want.float()[live], **_tol(dt))
    torch.testing.assert_close(st_dev.cpu(), st_ref, atol=1e-5, rtol=1e-5)     # slot 1 and the skipped sequence untouched


@pytest.mark.parametrize("dt", ACTS)
def test_scans_of_long_portions_run_in_segments(dt):
    """Portions longer than two segments of 32 rows take the three-pass form: same results, with a
    portion that starts from a kept state, one that starts at position 0, a short one and a skipped one."""
    g = torch.Generator().manual_seed(9)
    lens, starts = [300, 129, 5, 200], [40, 0, 7, 3]
    cu, pos, _ = _seqs(lens, starts)
    slots = torch.tensor([1, 0, 3, -1], dtype=torch.int32)
    T, w = int(cu[-1]), 70
    zxg = torch.randn(T, 3 * w, generator=g) * 2
    st = torch.randn(4, w, generator=g)
    st_ref = st.clone()
    want = ref.mingru_scan(zxg, st_ref, cu, pos, slots, dt)
    sd = st.to(DEV)
    got = ops.mingru_scan(zxg.to(DEV), sd, cu.to(DEV), pos.to(DEV), slots.to(DEV), dt, max_len=300)
    torch.testing.assert_close(got.float().cpu()[:434], want.float()[:434], **_tol(dt))
    torch.testing.assert_close(sd.cpu(), st_ref, atol=1e-5, rtol=1e-5)
    H, D, Dv = 2, 24, 70
    proj = torch.randn(T, 2 * H * D + 2 * H * Dv, generator=g)
    dec = torch.randn(T, H * D, generator=g) * 2 + 3
    st = torch.randn(4, H * D * Dv, generator=g)
    st_ref = st.clone()
    want = ref.gla_scan(proj, dec, st_ref, cu, pos, slots, H, D, Dv, 4.0)
    sd = st.to(DEV)
    got = ops.gla_scan(proj.to(DEV), dec.to(DEV), sd, cu.to(DEV), pos.to(DEV), slots.to(DEV), H, D, Dv, 4.0, max_len=300)
    torch.testing.assert_close(got.cpu()[:434], want[:434], atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(sd.cpu(), st_ref, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("H,D,Dv", [(2, 32, 32), (3, 24, 70), (1, 100, 8)])
def test_gla_scan_and_headnorm(H, D, Dv):
    g = torch.Generator().manual_seed(D)
    cu, pos, _ = _seqs([6, 1, 2], [0, 5, 3])
    slots = torch.tensor([1, 3, 0], dtype=torch.int32)
    T = 9
    proj = torch.randn(T, 2 * H * D + 2 * H * Dv + 5, generator=g)
    dec = torch.randn(T, H * D, generator=g) * 3
    st = torch.randn(4, H * D * Dv, generator=g)
    st_ref = st.clone()
    want = ref.gla_scan(proj, dec, st_ref, cu, pos, slots, H, D, Dv, 8.0)
    st_dev = st.to(DEV)
    pd = proj.to(DEV)
    got = ops.gla_scan(pd, dec.to(DEV), st_dev, cu.to(DEV), pos.to(DEV), slots.to(DEV), H, D, Dv, 8.0)
    torch.testing.assert_close(got.cpu(), want, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(st_dev.cpu(), st_ref, atol=1e-4, rtol=1e-4)
    wn = torch.rand(Dv, generator=g) + 0.5
    gate = proj[:, 2 * H * D + H * Dv:2 * H * D + 2 * H * Dv]
    for dt in ACTS:
        y = ops.headnorm_gate(got, wn.to(DEV), pd[:, 2 * H * D + H * Dv:2 * H * D + 2 * H * Dv], Dv, 1e-5, dt)
        torch.testing.assert_close(y.float().cpu(), ref.headnorm_gate(want, wn, gate, Dv, 1e-5, dt).float(), **_tol(dt))


@pytest.mark.parametrize("dt", ACTS)
@pytest.mark.parametrize("H,G,D,Dv,rot,chunk,window", [(4, 2, 32, 20, 8, 7, 0), (3, 3, 48, 72, 48, 0, 5), (2, 1, 16, 16, 0, 0, 0),
                                                       (6, 2, 96, 40, 24, 100, 0), (4, 2, 64, 48, 16, 40, 0),
                                                       (2, 2, 128, 128, 64, 0, 33)])
def test_qkv_prep_and_masked_attention(dt, H, G, D, Dv, rot, chunk, window):
    g = torch.Generator().manual_seed(H * 100 + D)
    BS, NB = 16, 24
    lens, starts = [150, 1, 37], [0, 70, 20]
    cu, pos, rs = _seqs(lens, starts)
    T = int(cu[-1])
    # block tables: distinct shuffled blocks per sequence
    perm = torch.randperm(NB, generator=g).tolist()
    need = [(s + n + BS - 1) // BS for n, s in zip(lens, starts)]
    bt = torch.zeros(3, max(need), dtype=torch.int32)
    at = 0
    for b, n in enumerate(need):
        bt[b, :n] = torch.tensor(perm[at:at + n], dtype=torch.int32)
        at += n
    slot = torch.tensor([int(bt[b, p // BS]) * BS + p % BS for b, p in zip(rs.tolist(), pos.tolist())], dtype=torch.int32)
    kc = torch.randn(NB, G, BS, D, generator=g).to(dt)        # "earlier" keys already in the cache
    vc = torch.randn(NB, G, BS, Dv, generator=g).to(dt)
    qkv = torch.randn(T, H * D + G * D + G * Dv + 3, generator=g)
    qn, kn = torch.rand(H * D, generator=g) + 0.5, torch.rand(G * D, generator=g) + 0.5
    half = rot // 2
    inv = torch.tensor([10000.0 ** (-2.0 * j / rot) for j in range(half)] or [0.0])
    kc_ref, vc_ref = kc.clone(), vc.clone()
    q_ref = ref.qkv_prep(qkv, qn, kn, pos, slot, kc_ref, vc_ref, H, G, D, Dv, rot, 10000.0, 1e-5)
    kd, vd = kc.to(DEV), vc.to(DEV)
    q = ops.qkv_prep(qkv.to(DEV), qn.to(DEV), kn.to(DEV), inv.to(DEV), pos.to(DEV), slot.to(DEV), kd, vd, H, G, D, Dv,
                     rot, 10000.0, 1e-5)
    torch.testing.assert_close(q.cpu(), q_ref, atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(kd.float().cpu(), kc_ref.float(), **_tol(dt))
    torch.testing.assert_close(vd.float().cpu(), vc_ref.float(), **_tol(dt))
    # a layer without keys of its own: queries only
    q2 = ops.qkv_prep(qkv[:, :H * D].contiguous().to(DEV), qn.to(DEV), None, inv.to(DEV), pos.to(DEV), slot.to(DEV),
                      None, None, H, G, D, Dv, rot, 10000.0, 1e-5)
    torch.testing.assert_close(q2.cpu(), q_ref, atol=2e-4, rtol=2e-4)
    want = ref.attn_masked(q_ref, kc_ref, vc_ref, bt, cu, pos, H, G, D, Dv, 0.3, chunk, window, torch.float32)
    got = ops.attn_masked(q, kd, vd, bt.to(DEV), cu.to(DEV), rs.to(DEV), pos.to(DEV), H, G, D, Dv, 0.3, chunk, window, dt)
    if ops.attn_tile_ok(D, Dv):
        # the same step with sequence 0 declared a prompt portion: fp32 MFMA tiles for its 150 rows,
        # the row kernel for the rest (a portion behind a single token is not a layout the engine
        # makes, so the other two stay rows)
        tiled = ops.attn_masked(q, kd, vd, bt.to(DEV), cu.to(DEV), rs.to(DEV), pos.to(DEV), H, G, D, Dv, 0.3, chunk,
                                window, dt, n_portions=1, portion_rows=150, max_len=150)
        torch.testing.assert_close(tiled.float().cpu(), want,
                                   **(_tol(dt) if dt == torch.bfloat16 else dict(atol=2e-4, rtol=2e-4)))
    torch.testing.assert_close(got.float().cpu(), want, **(_tol(dt) if dt == torch.bfloat16 else dict(atol=2e-4, rtol=2e-4)))


# ------------------------------------------------------------------ pre-norm designs, latent attention, mLSTM, routing
@pytest.mark.parametrize("dt", ACTS)
@pytest.mark.parametrize("T,d", [(3, 10), (600, 130)])
def test_scaled_embedding_with_positions_and_the_pre_norm_residual_step(dt, T, d):
    g = torch.Generator().manual_seed(T)
    E = torch.randn(37, d, generator=g).to(dt)
    ids = torch.randint(0, 37, (T,), generator=g).to(torch.int32)
    pos = torch.randint(0, 5000, (T,), generator=g).to(torch.int32)
    f = torch.tensor([10000.0 ** (-2.0 * i / d) for i in range(d // 2)], dtype=torch.float64)
    x, _ = ops.embed_rows(ids.to(DEV), E.to(DEV), None, None, 0.37, pos.to(DEV), f.to(DEV))
    xr, _ = ops.embed_rows(ids, E, None, None, 0.37, pos, f)
    torch.testing.assert_close(x.cpu(), xr, atol=2e-6, rtol=1e-6)       # angles of a few thousand radians, reduced in fp64
    y, w = torch.randn(T, d, generator=g), torch.rand(d, generator=g) + 0.5
    xa = ops.add_rmsnorm(x, y.to(DEV), w.to(DEV), 1e-3, dt)
    want = ref.add_rmsnorm(xr, y, w, 1e-3, dt)
    torch.testing.assert_close(x.cpu(), xr, atol=3e-4, rtol=1e-5)
    torch.testing.assert_close(xa.float().cpu(), want.float(), **(_tol(dt) if dt == torch.bfloat16 else dict(atol=3e-4, rtol=1e-4)))
    assert ops.add_rmsnorm(x, y.to(DEV), None, 1e-3, dt) is None         # the sum alone
    ref.add_rmsnorm(xr, y, None, 1e-3, dt)
    torch.testing.assert_close(x.cpu(), xr, atol=3e-4, rtol=1e-5)
    only = ops.add_rmsnorm(x, None, w.to(DEV), 1e-3, dt)                 # the norm alone
    torch.testing.assert_close(only.float().cpu(), ref.add_rmsnorm(xr, None, w, 1e-3, dt).float(),
                               **(_tol(dt) if dt == torch.bfloat16 else dict(atol=3e-4, rtol=1e-4)))


@pytest.mark.parametrize("dt", ACTS)
@pytest.mark.parametrize("R", [9, 64, 200])
def test_latent_write(dt, R):
    g = torch.Generator().manual_seed(R)
    T, BS, col0 = 11, 8, 5
    proj = torch.randn(T, col0 + R + 3, generator=g)
    w = torch.rand(R, generator=g) + 0.5
    slots = torch.tensor([3, 9, -1, 0, 17, 22, 23, 8, -1, 30, 31], dtype=torch.int32)
    c_ref = torch.zeros(4, 1, BS, R, dtype=dt)
    ref.latent_write(proj, col0, w, 1e-5, slots, c_ref)
    c = torch.zeros(4, 1, BS, R, dtype=dt, device=DEV)
    ops.latent_write(proj.to(DEV), col0, w.to(DEV), 1e-5, slots.to(DEV), c)
    torch.testing.assert_close(c.float().cpu(), c_ref.float(), **_tol(dt))


@pytest.mark.parametrize("a_dt,w_dt,o_dt", [(torch.float32, torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16, torch.bfloat16),
                                            (torch.float32, torch.float32, torch.float32)])
@pytest.mark.parametrize("M,H,N,K", [(1, 3, 7, 5), (70, 2, 130, 24), (5, 6, 64, 64)])
def test_head_linear(a_dt, w_dt, o_dt, M, H, N, K):
    g = torch.Generator().manual_seed(M + N)
    wide = torch.randn(M, H * K + H + 4, generator=g).to(a_dt)
    x = wide[:, 2:2 + H * K]                       # a column slice, as the model passes it
    W = (torch.randn(H, N, K, generator=g) / K ** 0.5).to(w_dt)
    gate = torch.randn(M, H + 3, generator=g)
    wd, gd = wide.to(DEV), gate.to(DEV)
    for gt, gtd in ((None, None), (gate[:, 1:1 + H], gd[:, 1:1 + H])):
        got = ops.head_linear(wd[:, 2:2 + H * K], W.to(DEV), o_dt, gtd)
        want = ref.head_linear(x, W, o_dt, gt)
        torch.testing.assert_close(got.float().cpu(), want.float(), **_tol(o_dt if a_dt == torch.float32 else torch.bfloat16))


def _mlstm_case(lens, starts, slots, H, D, Dv, cap, seed, max_len=1):
    g = torch.Generator().manual_seed(seed)
    cu, pos, _ = _seqs(lens, starts)
    slots = torch.tensor(slots, dtype=torch.int32)
    T = int(cu[-1])
    proj = torch.randn(T, 2 * H * D + 2 * H * Dv + 2 * H + 3, generator=g)
    proj[:, 2 * H * D + 2 * H * Dv:] *= 4                                      # gate logits that the cap bends
    st = torch.randn(4, H * D * (Dv + 1) + H, generator=g)
    st_ref = st.clone()
    o_ref, m_ref = ref.mlstm_scan(proj, st_ref, cu, pos, slots, H, D, Dv, cap)
    sd, pd = st.to(DEV), proj.to(DEV)
    o, m = ops.mlstm_scan(pd, sd, cu.to(DEV), pos.to(DEV), slots.to(DEV), H, D, Dv, cap, max_len=max_len)
    live = torch.cat([torch.arange(int(cu[b]), int(cu[b + 1])) for b in range(len(lens)) if int(slots[b]) >= 0])
    torch.testing.assert_close(o.cpu()[live], o_ref[live], atol=3e-4, rtol=3e-4)
    torch.testing.assert_close(m.cpu()[live], m_ref[live], atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(sd.cpu(), st_ref, atol=3e-4, rtol=3e-4)
    wn = torch.rand(H * Dv, generator=g) + 0.5
    c0 = 2 * H * D + H * Dv
    for dt in ACTS:
        y = ops.mlstm_out(o, m, wn.to(DEV), pd[:, c0:c0 + H * Dv], H, Dv, 1e-5, dt)
        want = ref.mlstm_out(o_ref, m_ref, wn, proj[:, c0:c0 + H * Dv], H, Dv, 1e-5, dt)
        torch.testing.assert_close(y.float().cpu()[live], want.float()[live],
                                   **(_tol(dt) if dt == torch.bfloat16 else dict(atol=2e-3, rtol=2e-3)))


@pytest.mark.parametrize("H,D,Dv,cap", [(2, 32, 32, 15.0), (3, 24, 70, 2.0), (1, 100, 8, 0.0), (5, 7, 63, 6.0), (2, 160, 40, 5.0)])
def test_mlstm_scan_and_read_out(H, D, Dv, cap):
    """Sequences that start at position 0 (zero state, maximum 0) and that continue from a kept state,
    a single decoded token, a skipped sequence; more than 64 rows (the maxima come from wave scans of 64)."""
    _mlstm_case([6, 1, 2, 150, 3], [0, 5, 3, 0, 9], [1, 3, 0, 2, -1], H, D, Dv, cap, seed=D)


def test_mlstm_long_portions_run_in_segments():
    _mlstm_case([300, 129, 5, 200], [40, 0, 7, 3], [1, 0, 3, -1], 2, 24, 70, 8.0, seed=5, max_len=300)


@pytest.mark.parametrize("dt", ACTS)
def test_glu(dt):
    y = torch.randn(13, 2 * 37, generator=torch.Generator().manual_seed(1))
    for kind in ("relu", "silu"):
        torch.testing.assert_close(ops.glu(y.to(DEV), dt, kind).float().cpu(), ref.glu(y, dt, kind).float(), **_tol(dt))


@pytest.mark.parametrize("n,top,groups,keep", [(20, 3, 5, 2), (8, 2, 1, 1), (70, 5, 7, 3), (130, 8, 10, 10), (12, 12, 4, 4), (6, 1, 6, 1)])
def test_route_grouped(n, top, groups, keep):
    g = torch.Generator().manual_seed(n)
    T = 75
    z = torch.randn(T, n, generator=g) * 2
    corr = torch.randn(n, generator=g) * 0.1 - 0.5                              # choice scores below zero
    ids, wts = ops.route_grouped(z.to(DEV), corr.to(DEV), top, groups, keep, 1.7)
    ids_ref, wts_ref = ref.route_grouped(z, corr, top, groups, keep, 1.7)
    assert (ids.cpu() == ids_ref).all()
    torch.testing.assert_close(wts.cpu(), wts_ref, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("x_dt,w_dt", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("T,top,E,I,d,ff", [(1, 2, 3, 1, 10, 7), (90, 3, 5, 2, 40, 20), (200, 4, 40, 0, 24, 70)])
def test_sorted_expert_products_and_mix(x_dt, w_dt, T, top, E, I, d, ff):
    g = torch.Generator().manual_seed(T)
    n = E + I
    ids = torch.stack([torch.randperm(n, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    wts = torch.rand(T, top, generator=g)
    x = torch.randn(T, d, generator=g).to(x_dt)
    up = (torch.randn(E, ff, d, generator=g) / d ** 0.5).to(w_dt)
    down = (torch.randn(E, d, ff, generator=g) / ff ** 0.5).to(w_dt)
    shared = torch.randn(T, d, generator=g)
    off, src, slot = ops.moe_sort(ids.to(DEV), n)
    off_ref, src_ref, slot_ref = ref_sort = ops.moe_sort(ids, n)
    assert (off.cpu() == off_ref).all()
    flat = ids.reshape(-1)
    sl = slot.cpu().long()
    assert sorted(sl.tolist()) == list(range(T * top))                                   # a permutation
    assert ((sl >= off.cpu()[flat.long()]) & (sl < off.cpu()[flat.long() + 1])).all()       # inside its expert's range
    assert (src.cpu()[sl] == torch.arange(T * top) // top).all()
    act = ops.grouped_linear(x.to(DEV), src, off, up.to(DEV), x_dt, T * top, relu2_epi=True)
    ye = ops.grouped_linear(act, None, off, down.to(DEV), torch.float32, T * top)
    got = ops.moe_mix(ye, slot, ids.to(DEV), wts.to(DEV), x.to(DEV), E, shared.to(DEV))
    act_ref = ref.grouped_linear(x, src_ref, off_ref, up, x_dt, T * top, relu2_epi=True)
    ye_ref = ref.grouped_linear(act_ref, None, off_ref, down, torch.float32, T * top)
    want = ref.moe_mix(ye_ref, slot_ref, ids, wts, x, E, shared)
    torch.testing.assert_close(got.cpu(), want, **(dict(atol=5e-2, rtol=5e-2) if x_dt == torch.bfloat16 else dict(atol=1e-4, rtol=1e-4)))
    none = ops.moe_mix(ye, slot, ids.to(DEV), wts.to(DEV), x.to(DEV), E, None)
    torch.testing.assert_close(none.cpu(), want - shared, **(dict(atol=5e-2, rtol=5e-2) if x_dt == torch.bfloat16 else dict(atol=1e-4, rtol=1e-4)))


@pytest.mark.parametrize("T,top,E,d,ff", [(5, 2, 3, 64, 64), (100, 3, 6, 128, 192), (400, 4, 9, 64, 128)])
def test_sorted_expert_products_on_the_packed_mfma_kernels(T, top, E, d, ff):
    """bf16 experts whose depths are multiples of 64 go through the grouped MFMA kernels (a panel per expert up to a few
    hundred routed rows, tiles beyond) with the relu^2 and fp32 epilogues; experts past E get no rows written."""
    g = torch.Generator().manual_seed(T)
    n = E + 2
    ids = torch.stack([torch.randperm(n, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    x = torch.randn(T, d, generator=g).to(torch.bfloat16)
    up = (torch.randn(E, ff, d, generator=g) / d ** 0.5).to(torch.bfloat16)
    down = (torch.randn(E, d, ff, generator=g) / ff ** 0.5).to(torch.bfloat16)
    off, src, slot = ops.moe_sort(ids.to(DEV), n)
    act = ops.grouped_linear(x.to(DEV), src, off, ops.ExpertWeights.from_dense(up, DEV), torch.bfloat16, T * top, relu2_epi=True)
    ye = ops.grouped_linear(act, None, off, ops.ExpertWeights.from_dense(down, DEV), torch.float32, T * top)
    act_ref = ref.grouped_linear(x, src.cpu(), off.cpu(), up, torch.bfloat16, T * top, relu2_epi=True)
    ye_ref = ref.grouped_linear(act_ref, None, off.cpu(), down, torch.float32, T * top)
    real = int(off.cpu()[E])
    torch.testing.assert_close(act.float().cpu()[:real], act_ref.float()[:real], atol=3e-2, rtol=3e-2)
    torch.testing.assert_close(ye.cpu()[:real], ye_ref[:real], atol=3e-2, rtol=3e-2)


# ---- Dynamic Tanh residual step, neighbouring rotary pairs with keys as values, clamped gated units ----
@pytest.mark.parametrize("dt", ACTS)
@pytest.mark.parametrize("T,d", [(3, 10), (600, 132), (1, 64)])
def test_dynamic_tanh_residual_step(dt, T, d):
    g = torch.Generator().manual_seed(T + d)
    x0, y = torch.randn(T, d, generator=g), torch.randn(T, d, generator=g)
    w, b = torch.randn(d, generator=g), torch.randn(d, generator=g)
    x = x0.clone().to(DEV)
    xa = ops.add_dyt(x, y.to(DEV), 0.7, 0.4, w.to(DEV), b.to(DEV), dt)
    xr = x0.clone()
    want = torch.empty(T, d, dtype=dt)
    ref.add_dyt(xr, y, 0.7, 0.4, w, b, want)
    torch.testing.assert_close(x.cpu(), xr, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(xa.float().cpu(), want.float(), **_tol(dt))
    # the norm alone leaves the stream as it is; the sum alone returns nothing
    x2 = x0.clone().to(DEV)
    torch.testing.assert_close(ops.add_dyt(x2, None, 0.7, 0.4, w.to(DEV), b.to(DEV), dt).float().cpu(),
                               (torch.tanh(0.4 * x0) * w + b).to(dt).float(), **_tol(dt))
    torch.testing.assert_close(x2.cpu(), x0)
    assert ops.add_dyt(x2, y.to(DEV), 2.0, 1.0, None, None, None) is None
    torch.testing.assert_close(x2.cpu(), x0 + 2.0 * y)
    # the stream itself, cast, into the left and the right half of a wider matrix
    both = torch.zeros(T, 2 * d, dtype=dt, device=DEV)
    ops.add_dyt(x2, None, 1.0, 1.0, None, None, dt, out=both[:, d:])
    ops.add_dyt(x2, y.to(DEV), -2.0, 1.0, None, None, dt, out=both[:, :d])
    torch.testing.assert_close(both.float().cpu(), torch.cat([x0, x0 + 2.0 * y], 1).to(dt).float(), **_tol(dt))


@pytest.mark.parametrize("dt", ACTS)
@pytest.mark.parametrize("H,G,D,rot,window", [(4, 2, 32, 8, 7), (3, 3, 48, 48, 40), (2, 1, 16, 0, 5), (5, 1, 7, 6, 3), (6, 3, 64, 16, 100)])
def test_rotary_pairs_keys_as_values_and_window_attention(dt, H, G, D, rot, window):
    g = torch.Generator().manual_seed(H * 100 + D)
    lens, starts = [37, 70, 1, 1], [0, 130, 55, 3]          # two portions (one continuing at place 130), two decoded tokens
    BSZ, MB = 16, 14
    cu, pos, rs = _seqs(lens, starts)
    T = int(cu[-1])
    tables = torch.randperm(4 * MB, generator=g).to(torch.int32).view(4, MB)
    slots = torch.tensor([int(tables[b, p // BSZ]) * BSZ + p % BSZ for b, p in zip(rs.tolist(), pos.tolist())], dtype=torch.int32)
    qk = torch.randn(T, (H + G) * D + 5, generator=g)
    base = (torch.randn(4 * MB, G, BSZ, D, generator=g) * 0.5).to(dt)        # what earlier steps left in the pages
    inv = torch.tensor([1e4 ** (-2.0 * j / rot) for j in range(rot // 2)], dtype=torch.float64) if rot else None
    kc, vc = base.clone(), (base.clone() * 0.7 if rot else None)
    kd, vd = kc.clone().to(DEV), (vc.clone().to(DEV) if rot else None)
    q = ops.rope_pairs_write(qk.to(DEV), inv.to(DEV) if rot else None, pos.to(DEV), slots.to(DEV), kd, vd, H, G, D, rot)
    qr = ref.rope_pairs_write(qk, inv, pos, slots, kc, vc, H, G, D, rot)
    torch.testing.assert_close(q.cpu(), qr, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(kd.float().cpu(), kc.float(), **_tol(dt))
    if rot:
        torch.testing.assert_close(vd.float().cpu(), vc.float(), **_tol(dt))
    vv, vvd = (vc, vd) if rot else (kc, kd)
    want = ref.attn_masked(qr, kc, vv, tables, cu, pos, H, G, D, D, 0.2, 0, window, dt)
    for portions, rows in ((0, 0), (2, 107)):               # the row kernel for everything; matrix-core tiles for the portions
        got = ops.attn_masked(q, kd, vvd, tables.to(DEV), cu.to(DEV), rs.to(DEV), pos.to(DEV), H, G, D, D, 0.2, 0, window, dt,
                              n_portions=portions, portion_rows=rows, max_len=70)
        torch.testing.assert_close(got.float().cpu(), want.float(), **_tol(dt))


@pytest.mark.parametrize("dt", ACTS)
def test_clamped_gated_unit(dt):
    g = torch.Generator().manual_seed(5)
    y = torch.randn(33, 50, generator=g) * 2
    got = ops.glu_clamped(y.to(DEV), 3, 20, 17, 0.8, dt)
    gate, up = y[:, 3:20].clamp(max=0.8), y[:, 20:37].clamp(-0.8, 0.8)
    torch.testing.assert_close(got.float().cpu(), (gate * torch.sigmoid(1.702 * gate) * (up + 1)).to(dt).float(), **_tol(dt))
    # a work list: entry r names row slot_of[r], scaled by wts[r] BEFORE the clamps
    slot_of = torch.randperm(33, generator=g).to(torch.int32)
    wts = torch.rand(33, generator=g)
    got = ops.glu_clamped(y.to(DEV), 0, 25, 25, 1.5, dt, slot_of=slot_of.to(DEV), wts=wts.to(DEV), slope=1.1, shift=0.5)
    s = torch.empty(33)
    s[slot_of.long()] = wts
    gate, up = (y[:, :25] * s[:, None]).clamp(max=1.5), (y[:, 25:] * s[:, None]).clamp(-1.5, 1.5)
    torch.testing.assert_close(got.float().cpu(), (gate * torch.sigmoid(1.1 * gate) * (up + 0.5)).to(dt).float(), **_tol(dt))
    torch.testing.assert_close(ref.glu_clamped(y, 0, 25, 25, 1.5, 1.1, 0.5, slot_of, wts, dt, 33).float(), got.float().cpu(), **_tol(dt))


@pytest.mark.parametrize("n,top", [(6, 2), (70, 5), (3, 3), (130, 1)])
def test_route_by_sigmoid_scores(n, top):
    g = torch.Generator().manual_seed(n)
    z = torch.randn(50, n + 3, generator=g)[:, 1:n + 1]           # a column slice of a wider matrix
    ids, wts = ops.route_grouped(z.to(DEV), None, top, 1, 1, 1.0, score="sigmoid")
    ri, rw = ref.route_grouped(z, None, top, 1, 1, 1.0, "sigmoid")
    assert (ids.cpu() == ri).all()
    torch.testing.assert_close(wts.cpu(), rw, atol=1e-6, rtol=1e-5)
    torch.testing.assert_close(rw, torch.sigmoid(z).gather(1, ri.long()))


def test_expert_mix_without_weights_under_a_gated_shared_expert():
    g = torch.Generator().manual_seed(2)
    T, top, E, d = 40, 3, 7, 24
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    offsets, src, slot_of = ops.moe_sort(ids.to(DEV), E)
    ye, shared, h = torch.randn(T * top, d, generator=g), torch.randn(T, d, generator=g), torch.randn(T, d, generator=g)
    wide = torch.randn(T, 9, generator=g)
    got = ops.moe_mix(ye.to(DEV), slot_of, ids.to(DEV), None, h.to(DEV), E, shared.to(DEV), wide.to(DEV)[:, 4:5])
    want = ye[slot_of.cpu().long()].view(T, top, d).sum(1) + torch.sigmoid(wide[:, 4:5]) * shared
    torch.testing.assert_close(got.cpu(), want, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("T,top,E,d,ff", [(5, 2, 3, 64, 64), (100, 3, 6, 128, 192), (400, 4, 9, 64, 128), (33, 1, 40, 64, 32)])
def test_clamped_gated_experts_as_the_epilogue_of_the_packed_product(T, top, E, d, ff):
    """The gate | up product of every expert on the MFMA kernels (one panel per expert for few rows, tiles beyond) with
    the clamped gated unit and the per-row scale in its epilogue, against the plain product and unit."""
    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, d, generator=g).to(torch.bfloat16)
    gate = (torch.randn(E, ff, d, generator=g) * 2 / d ** 0.5).to(torch.bfloat16)
    up = (torch.randn(E, ff, d, generator=g) * 2 / d ** 0.5).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    wts = torch.rand(T, top, generator=g)
    offsets, src, slot_of, sw = ops.moe_sort(ids.to(DEV), E, wts.to(DEV))
    torch.testing.assert_close(sw.cpu()[slot_of.cpu().long()], wts.reshape(-1))
    W = ops.ExpertWeights.from_dense(torch.stack([ops.interleave_gate_up(gate[e], up[e]) for e in range(E)]), DEV, swiglu=True)
    got = ops.grouped_linear(x.to(DEV), src, offsets, W, torch.bfloat16, T * top, glu_clamp=(sw, 0.6, 1.702, 1.0))
    plain = ref.grouped_linear(x, src.cpu(), offsets.cpu(), torch.cat([gate, up], 1), torch.float32, T * top)
    want = ref.glu_clamped(plain, 0, ff, ff, 0.6, 1.702, 1.0, slot_of.cpu(), wts.reshape(-1), torch.float32, T * top)
    torch.testing.assert_close(got.float().cpu(), want, atol=2e-2, rtol=2e-2)
    with pytest.raises(ValueError):
        ops.grouped_linear(x.to(DEV), src, offsets, W, torch.float32, T * top)


# ------------------------------------------------------------------ parallel residual streams, turned values, mixed heads'
# weights, a turned key part beside the latent row, xIELU (hybrid_streams.hip; options of the attention kernels)
@pytest.mark.parametrize("dt", ACTS)
@pytest.mark.parametrize("T,S,d", [(3, 1, 10), (7, 3, 72), (600, 2, 130), (5, 8, 257), (700, 4, 64)])
def test_parallel_streams_start_and_sublayer_step(dt, T, S, d):
    g = torch.Generator().manual_seed(T + S)
    x0, w = torch.randn(T, d, generator=g) * 3, torch.rand(d, generator=g) + 0.5
    xs = ops.hc_init(x0.to(DEV), w.to(DEV), 1e-3, S)
    xr = ref.hc_init(x0, w, 1e-3, S)
    torch.testing.assert_close(xs.cpu(), xr, atol=1e-5, rtol=1e-5)
    xs = (xs + 0.3 * torch.randn(T, S, d, generator=g).to(DEV)).contiguous()          # streams that have grown apart
    xr = xs.cpu().clone()
    mix, ow, iw = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
    nw, y = torch.rand(d, generator=g) + 0.5, torch.randn(T, d, generator=g)
    tol = _tol(dt) if dt == torch.bfloat16 else dict(atol=2e-5, rtol=2e-5)
    # the read alone (the first sublayer of a step), normed
    a = ops.hc_step(xs, None, None, None, iw.to(DEV), nw.to(DEV), 1e-3, dt)
    torch.testing.assert_close(a.float().cpu(), ref.hc_step(xr, None, None, None, iw, nw, 1e-3, dt).float(), **tol)
    torch.testing.assert_close(xs.cpu(), xr)
    # write and read, normed
    a = ops.hc_step(xs, y.to(DEV), mix.to(DEV), ow.to(DEV), iw.to(DEV), nw.to(DEV), 1e-3, dt)
    want = ref.hc_step(xr, y, mix, ow, iw, nw, 1e-3, dt)
    torch.testing.assert_close(xs.cpu(), xr, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(a.float().cpu(), want.float(), **tol)
    # write, and the plain combination in fp32 (the model's output: every stream once)
    ones = torch.ones(S)
    u = ops.hc_step(xs, y.to(DEV), mix.to(DEV), ow.to(DEV), ones.to(DEV), None, 1e-3, None)
    want = ref.hc_step(xr, y, mix, ow, ones, None, 1e-3, None)
    assert u.dtype == torch.float32
    torch.testing.assert_close(xs.cpu(), xr, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(u.cpu(), want, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(want, xr.sum(1), atol=1e-4, rtol=1e-4)
    # the write alone
    assert ops.hc_step(xs, y.to(DEV), mix.to(DEV), ow.to(DEV), None, None, 1e-3, None) is None
    ref.hc_step(xr, y, mix, ow, None, None, 1e-3, None)
    torch.testing.assert_close(xs.cpu(), xr, atol=1e-3, rtol=1e-4)


@pytest.mark.parametrize("dt", ACTS)
@pytest.mark.parametrize("H,G,D,Dv,rot,pairs,window,cap", [(4, 2, 32, 32, 8, False, 7, 3.0), (3, 3, 48, 16, 48, False, 40, 0.0), (2, 1, 16, 48, 0, False, 5, 50.0),
                                                           (5, 1, 7, 6, 6, True, 3, 1.5), (8, 4, 16, 64, 16, False, 100, 20.0), (6, 3, 24, 200, 8, True, 30, 2.0)])
def test_turned_values_capped_scores_a_sink_and_mixed_heads(dt, H, G, D, Dv, rot, pairs, window, cap):
    g = torch.Generator().manual_seed(H * 100 + D)
    lens, starts = [37, 70, 1, 1], [0, 130, 55, 3]          # two portions (one continuing at place 130), two decoded tokens
    BSZ, MB = 16, 14
    cu, pos, rs = _seqs(lens, starts)
    T = int(cu[-1])
    tables = torch.randperm(4 * MB, generator=g).to(torch.int32).view(4, MB)
    slots = torch.tensor([int(tables[b, p // BSZ]) * BSZ + p % BSZ for b, p in zip(rs.tolist(), pos.tolist())], dtype=torch.int32)
    qkv = torch.randn(T, H * D + G * (D + Dv) + 5, generator=g)
    kc, vc = (torch.randn(4 * MB, G, BSZ, D, generator=g) * 0.5).to(dt), (torch.randn(4 * MB, G, BSZ, Dv, generator=g) * 0.5).to(dt)
    inv = torch.tensor([1e3 ** (-2.0 * j / rot) for j in range(rot // 2)], dtype=torch.float64) if rot else None
    inv_v = torch.tensor([1e3 ** (-2.0 * j / Dv) for j in range(Dv // 2)], dtype=torch.float64)
    kd, vd = kc.clone().to(DEV), vc.clone().to(DEV)
    q = ops.rope_qkv_write(qkv.to(DEV), inv.to(DEV) if rot else None, inv_v.to(DEV), pos.to(DEV), slots.to(DEV), kd, vd, H, G, D, Dv,
                           rot, pairs, pairs)
    qr = ref.rope_qkv_write(qkv, inv, inv_v, pos, slots, kc, vc, H, G, D, Dv, rot, pairs, pairs)
    torch.testing.assert_close(q.cpu(), qr, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(kd.float().cpu(), kc.float(), **_tol(dt))
    torch.testing.assert_close(vd.float().cpu(), vc.float(), **_tol(dt))
    talk = torch.eye(H) + 0.5 * torch.randn(H, H, generator=g)
    for sink in (True, False):
        want = ref.attn_masked(qr, kc, vc, tables, cu, pos, H, G, D, Dv, 0.2, 0, window, torch.float32, cap, sink, True)
        assert want.shape == (T, H * G * Dv)
        mixed = ref.talk_mix(want, talk, pos, inv_v, H, G, Dv, dt, pairs)
        for portions, rows in ((0, 0), (2, 107)):               # the row kernel for everything; matrix-core tiles for the portions
            got = ops.attn_masked(q, kd, vd, tables.to(DEV), cu.to(DEV), rs.to(DEV), pos.to(DEV), H, G, D, Dv, 0.2, 0, window,
                                  torch.float32, n_portions=portions, portion_rows=rows, max_len=70, softcap=cap, sink=sink,
                                  all_value_heads=True)
            torch.testing.assert_close(got.cpu(), want, **(_tol(dt) if dt == torch.bfloat16 else dict(atol=2e-5, rtol=2e-5)))
            out = ops.talk_mix(got, talk.to(DEV), pos.to(DEV), inv_v.to(DEV), H, G, Dv, dt, pairs)
            torch.testing.assert_close(out.float().cpu(), mixed.float(), **(_tol(dt) if dt == torch.bfloat16 else dict(atol=5e-5, rtol=5e-5)))
        # each head on its own group's values only, under the same cap and sink
        own = ref.attn_masked(qr, kc, vc, tables, cu, pos, H, G, D, Dv, 0.2, 0, window, dt, cap, sink, False)
        got = ops.attn_masked(q, kd, vd, tables.to(DEV), cu.to(DEV), rs.to(DEV), pos.to(DEV), H, G, D, Dv, 0.2, 0, window, dt,
                              n_portions=2, portion_rows=107, max_len=70, softcap=cap, sink=sink)
        torch.testing.assert_close(got.float().cpu(), own.float(), **_tol(dt))
    # the mix alone, nothing turned back
    no_turn = ops.talk_mix(want.to(DEV), talk.to(DEV), pos.to(DEV), None, H, G, Dv, dt)
    torch.testing.assert_close(no_turn.float().cpu(), ref.talk_mix(want, talk, pos, None, H, G, Dv, dt, False).float(),
                               **(_tol(dt) if dt == torch.bfloat16 else dict(atol=5e-5, rtol=5e-5)))


@pytest.mark.parametrize("dt", ACTS)
@pytest.mark.parametrize("H,D,R,rd,Dv,window,own", [(4, 16, 24, 8, 16, 9, True), (3, 10, 20, 6, 14, 40, True), (2, 70, 130, 80, 66, 100, False),
                                                   (8, 64, 96, 32, 64, 33, True), (1, 5, 7, 2, 3, 4, True), (5, 8, 48, 0, 16, 12, True)])
def test_latent_rows_with_a_turned_key_part_shared_by_the_heads(dt, H, D, R, rd, Dv, window, own):
    g = torch.Generator().manual_seed(H * 100 + R)
    lens, starts = [37, 70, 1, 1], [0, 130, 55, 3]
    BSZ, MB = 16, 14
    cu, pos, rs = _seqs(lens, starts)
    T, W = int(cu[-1]), R + rd
    tables = torch.randperm(4 * MB, generator=g).to(torch.int32).view(4, MB)
    slots = torch.tensor([int(tables[b, p // BSZ]) * BSZ + p % BSZ for b, p in zip(rs.tolist(), pos.tolist())], dtype=torch.int32)
    nq = H * (D + rd)
    proj = torch.randn(T, nq + W + H * Dv + 3, generator=g)
    w = torch.rand(R, generator=g) + 0.5
    inv = torch.tensor([1e4 ** (-2.0 * j / rd) for j in range(rd // 2)], dtype=torch.float64) if rd else None
    cache = (torch.randn(4 * MB, 1, BSZ, W, generator=g) * 0.5).to(dt)
    cd = cache.clone().to(DEV)
    Uk = (torch.randn(H, R, D, generator=g) / D ** 0.5).to(dt)
    Uv = (torch.randn(H, Dv, R, generator=g) / R ** 0.5).to(dt)
    qlat_r = torch.zeros(T, H * W)
    ref.latent_rope_write(proj, nq, w, 1e-5, inv, pos, slots, cache if own else None, qlat_r, H, D, R, rd, True)
    ref.head_linear(proj, Uk, torch.float32, None, D + rd, qlat_r, W)
    qlat = torch.zeros(T, H * W, device=DEV)
    ops.latent_rope_write(proj.to(DEV), nq, w.to(DEV), 1e-5, inv.to(DEV) if rd else None, pos.to(DEV), slots.to(DEV),
                          cd if own else None, qlat, H, D, R, rd)
    ops.head_linear(proj.to(DEV), Uk.to(DEV), torch.float32, x_head_stride=D + rd, out=qlat, out_head_stride=W)
    torch.testing.assert_close(qlat.cpu(), qlat_r, atol=3e-5, rtol=3e-5)
    torch.testing.assert_close(cd.float().cpu(), cache.float(), **_tol(dt))
    # the cached rows are the keys; their first R columns are the values
    want = ref.attn_masked(qlat_r, cache, cache[..., :R], tables, cu, pos, H, 1, W, R, 0.2, 0, window, torch.float32)
    gate = proj[:, nq + W:nq + W + H * Dv]
    o_ref = ref.head_linear(want, Uv, dt, gate, gate_full=True)
    for portions, rows in ((0, 0), (2, 107)):
        got = ops.attn_masked(qlat, cd, cd[..., :R], tables.to(DEV), cu.to(DEV), rs.to(DEV), pos.to(DEV), H, 1, W, R, 0.2, 0, window,
                              torch.float32, n_portions=portions, portion_rows=rows, max_len=70)
        torch.testing.assert_close(got.cpu(), want, **(_tol(dt) if dt == torch.bfloat16 else dict(atol=3e-5, rtol=3e-5)))
        o = ops.head_linear(got, Uv.to(DEV), dt, gate=proj.to(DEV)[:, nq + W:nq + W + H * Dv], gate_full=True)
        torch.testing.assert_close(o.float().cpu(), o_ref.float(), **(_tol(dt) if dt == torch.bfloat16 else dict(atol=5e-5, rtol=5e-5)))


@pytest.mark.parametrize("dt", ACTS)
def test_xielu(dt):
    g = torch.Generator().manual_seed(5)
    y = torch.randn(33, 50, generator=g) * 3
    for ap, an in ((0.8, 1.3), (0.0, 0.5), (2.5, 4.0)):
        got = ops.xielu(y.to(DEV)[:, 3:40], ap, an, dt)
        z = y[:, 3:40].double()
        want = torch.where(z > 0, ap * z * z + z / 2, an * (torch.exp(z) - 1 - z) + z / 2)
        torch.testing.assert_close(got.float().cpu(), want.float().to(dt).float(), **_tol(dt))
        torch.testing.assert_close(ref.xielu(y[:, 3:40], ap, an, dt).float(), got.float().cpu(), **_tol(dt))
