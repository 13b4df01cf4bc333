"""HIP kernels of the hybrid decoders against their fp32 PyTorch references
(``ops.reference``), op by op, in bf16 and fp32, on sizes that are not multiples of the
wave (odd head sizes, several norm groups, chunks that continue a slot's state)."""
import types

import pytest
import torch

from kubernetes_gpu_cluster_amd import ops
from kubernetes_gpu_cluster_amd.ops import reference as ref

pytestmark = pytest.mark.gpu
DT = [torch.bfloat16, torch.float32]


def _tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("W,G", [(352, 2), (384, 3), (1024, 1)])
def test_group_norm_and_add(gpu, dt, W, G):
    torch.manual_seed(0)
    x = torch.randn(37, W) * 3
    y = torch.randn(37, W).to(dt)
    w = torch.rand(W) + 0.5
    want_x = x + y.float()
    want = ref.group_rms_norm(want_x, w, G, 1e-5, dt)
    xg = x.to(gpu)
    got = ops.group_rms_norm(xg, w.to(gpu), G, 1e-5, dt, add=y.to(gpu))
    torch.testing.assert_close(xg.cpu(), want_x)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))
    got2 = ops.group_rms_norm(xg, w.to(gpu), G, 1e-5, dt)
    torch.testing.assert_close(got2.cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DT)
def test_depth_mix_norm(gpu, dt):
    torch.manual_seed(1)
    L, cap, T, W, G, layer = 5, 16, 11, 192, 3, 3
    hist = torch.randn(L + 1, cap, W)
    x = torch.randn(T, W)
    y = torch.randn(T, W).to(dt)
    coef = torch.randn(layer + 2)
    w = torch.rand(W) + 0.5
    h_ref, x_ref = hist.clone(), x.clone()
    want = ops.depth_mix_norm(x_ref, h_ref, layer, y, coef, w, G, 1e-5, dt)
    hg, xg = hist.to(gpu), x.to(gpu)
    got = ops.depth_mix_norm(xg, hg, layer, y.to(gpu), coef.to(gpu), w.to(gpu), G, 1e-5, dt)
    torch.testing.assert_close(hg.cpu(), h_ref, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(xg.cpu(), x_ref, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DT)
def test_xielu_gate_proj_head_norm(gpu, dt):
    torch.manual_seed(2)
    z = (torch.randn(9, 200) * 3).to(dt)
    ab = torch.tensor([0.7, 1.3])
    torch.testing.assert_close(ops.xielu(z.to(gpu), ab.to(gpu)).cpu().float(),
                               ref.xielu(z, ab).float(), **_tol(dt))
    h = torch.randn(13, 288).to(dt)
    w = (torch.randn(10, 288) * 0.2).to(dt)
    b = torch.randn(10)
    want = ref.gate_proj(h, w, b, ops.GATE_CAP_TANH, ops.GATE_LOGSIG_CAP_TANH, 5, 15.0)
    got = ops.gate_proj(h.to(gpu), w.to(gpu), b.to(gpu), ops.GATE_CAP_TANH,
                        ops.GATE_LOGSIG_CAP_TANH, 5, 15.0)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-4)
    got = ops.gate_proj(h.to(gpu), w.to(gpu), None, ops.GATE_SIGMOID)
    torch.testing.assert_close(got.cpu(), ref.gate_proj(h, w, None, 0, 0, 10, 1.0), rtol=1e-4,
                               atol=1e-4)
    H, dv = 3, 40
    o = torch.randn(7, H * dv) * 5
    big = torch.randn(7, 300).to(dt)
    g = big[:, 100:100 + H * dv]
    nw = torch.rand(H * dv) + 0.5
    want = ref.head_norm_gate(o, g, nw, H, 1e-5, dt)
    got = ops.head_norm_gate(o.to(gpu), big.to(gpu)[:, 100:100 + H * dv], nw.to(gpu), H, 1e-5, dt)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))


def _meta(P_q, P_sl, D_ctx, tables, slots=None):
    """AttnMetadata stand-in: prefill chunks (query lens, seq lens) then decode rows."""
    m = types.SimpleNamespace()
    P, D = len(P_q), len(D_ctx)
    m.num_prefills, m.num_decodes, m.num_prefill_tokens = P, D, sum(P_q)
    qsl = [0]
    for q in P_q:
        qsl.append(qsl[-1] + q)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32)   # noqa: E731
    m.query_start_loc = i32(qsl) if P else None
    m.prefill_seq_lens = i32(P_sl) if P else None
    m.prefill_block_tables = tables[:P].contiguous() if P else None
    m.decode_ctx_lens = i32(D_ctx) if D else None
    m.decode_block_tables = tables[P:P + D].contiguous() if D else None
    m.state_slots = i32(slots) if slots is not None else None
    return m


def _to(m, dev):
    out = types.SimpleNamespace(**vars(m))
    for k, v in vars(m).items():
        if torch.is_tensor(v):
            setattr(out, k, v.to(dev))
    return out


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("H,G,dk,dv,rot,window,keep", [(6, 2, 40, 24, 16, 9, 3), (4, 4, 64, 64, 64, 0, 0),
                                                        (8, 1, 96, 128, 32, 70, 5)])
def test_rope_store_and_window_attention(gpu, dt, H, G, dk, dv, rot, window, keep):
    torch.manual_seed(3)
    bs, nb = 8, 64
    # two prefill chunks (one continuing at position 50, one fresh) and two decode rows
    P_q, P_sl, D_ctx = [13, 21], [63, 21], [90, 7]
    T = sum(P_q) + len(D_ctx)
    perm = torch.randperm(nb - 1)[:4 * 12].view(4, 12) + 1
    tables = perm.to(torch.int32)
    kc = torch.randn(nb, G, bs, dk).to(dt)
    vc = torch.randn(nb, G, bs, dv).to(dt)
    m = _meta(P_q, P_sl, D_ctx, tables)
    pos = torch.cat([torch.arange(50, 63), torch.arange(0, 21), torch.tensor([89, 6])])
    seq_of = [0] * 13 + [1] * 21 + [2, 3]
    slots = torch.tensor([int(tables[s, p // bs]) * bs + p % bs for s, p in zip(seq_of, pos.tolist())])
    qkv = torch.randn(T, (H + G) * dk + G * dv).to(dt)
    table = ref.rope_table(rot, 128, 10000.0)
    gate = torch.rand(T, H)
    kc_r, vc_r = kc.clone(), vc.clone()
    q_r = ops.rope_kv_store(qkv, pos, table, kc_r, vc_r, slots, H, G, dk, dv)
    want = ops.window_attention(q_r, kc_r, vc_r, pos, m, 0.11, window, keep, gate)
    kc_g, vc_g = kc.to(gpu), vc.to(gpu)
    q_g = ops.rope_kv_store(qkv.to(gpu), pos.to(gpu), table.to(gpu), kc_g, vc_g, slots.to(gpu),
                            H, G, dk, dv)
    tol = _tol(dt)
    torch.testing.assert_close(q_g.cpu().float(), q_r.float(), **tol)
    torch.testing.assert_close(kc_g.cpu().float(), kc_r.float(), **tol)
    torch.testing.assert_close(vc_g.cpu().float(), vc_r.float(), rtol=0, atol=0)
    got = ops.window_attention(q_r.to(gpu), kc_r.to(gpu), vc_r.to(gpu), pos.to(gpu), _to(m, gpu),
                               0.11, window, keep, gate.to(gpu))
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol)


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("H,d,dv", [(3, 24, 40), (2, 80, 64), (1, 136, 200)])
def test_mlstm_scan(gpu, dt, H, d, dv):
    torch.manual_seed(4)
    slots_n = 5
    # chunk continuing slot 3 (position 17), fresh chunk in slot 0, a padding sequence
    # (slot -1), decode rows continuing slots 4 and 1 (one of them at position 0)
    P_q, P_sl, D_ctx = [9, 14, 4], [26, 14, 4], [31, 1]
    slot_ids = [3, 0, -1, 4, 1]
    T = sum(P_q) + len(D_ctx)
    m = _meta(P_q, P_sl, D_ctx, torch.zeros(5, 1, dtype=torch.int32), slot_ids)
    S = torch.randn(slots_n, H, d, dv) * 0.3
    n = torch.randn(slots_n, H, d) * 0.3
    mm = torch.rand(slots_n, H) * 2
    qkvg = torch.randn(T, 2 * H * d + 2 * H * dv).to(dt)
    gates = torch.cat([torch.randn(T, H) * 2, -torch.rand(T, H) * 2], dim=1)
    st_r = (S.clone(), n.clone(), mm.clone())
    want = ops.mlstm_scan(qkvg, gates, st_r, m, H, d, dv)
    st_g = (S.to(gpu), n.to(gpu), mm.to(gpu))
    got = ops.mlstm_scan(qkvg.to(gpu), gates.to(gpu), st_g, _to(m, gpu), H, d, dv)
    torch.testing.assert_close(got.cpu(), want, rtol=2e-4, atol=2e-4)
    for a, b in zip(st_g, st_r):
        torch.testing.assert_close(a.cpu(), b, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("path", ["fast", "simple"])
@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("H,G,dk,dv,window,keep", [(4, 2, 96, 64, 70, 5), (4, 1, 128, 128, 150, 3),
                                                   (4, 2, 64, 32, 0, 0), (2, 1, 160, 96, 64, 70),
                                                   (3, 3, 32, 16, 1, 0), (6, 1, 64, 48, 129, 1)])
def test_window_attention_long_chunks(gpu, dt, path, H, G, dk, dv, window, keep, monkeypatch):
    """Chunks that span several 64-key tiles and 64-row blocks, continue long contexts and
    start mid-page, next to decode rows (one of them the first token of its sequence): the
    MFMA tile kernel and the 8-wave decode kernel (and, with KGC_WINDOW_ATTN=simple, the
    one-wave kernel alone) against the fp32 reference."""
    monkeypatch.setenv("KGC_WINDOW_ATTN", path)
    torch.manual_seed(5)
    bs = 8
    P_q, P_sl, D_ctx = [200, 77, 130], [300, 77, 513], [400, 65, 1]
    lens = P_sl + D_ctx
    mb = max(lens) // bs + 1
    nb = len(lens) * mb + 1
    tables = (torch.randperm(nb - 1)[: len(lens) * mb].view(len(lens), mb) + 1).to(torch.int32)
    kc = (torch.randn(nb, G, bs, dk) * 0.7).to(dt)
    vc = torch.randn(nb, G, bs, dv).to(dt)
    m = _meta(P_q, P_sl, D_ctx, tables)
    T = sum(P_q) + len(D_ctx)
    q = torch.randn(T, H, dk).to(dt)
    pos = torch.cat([torch.arange(sl - ql, sl) for ql, sl in zip(P_q, P_sl)] +
                    [torch.tensor([c - 1 for c in D_ctx])])
    gate = torch.rand(T, H)
    want = ops.window_attention(q, kc, vc, pos, m, 0.13, window, keep, gate)
    got = ops.window_attention(q.to(gpu), kc.to(gpu), vc.to(gpu), pos.to(gpu), _to(m, gpu), 0.13,
                               window, keep, gate.to(gpu))
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("rows,W,N", [(1500, 288, 10), (2048, 1536, 8), (1100, 2304, 19)])
def test_gate_proj_many_rows(gpu, dt, rows, W, N):
    """The row-blocked kernel (weights held in registers, >= 1024 rows)."""
    torch.manual_seed(6)
    h = torch.randn(rows, W).to(dt)
    w = (torch.randn(N, W) * 0.1).to(dt)
    b = torch.randn(N)
    want = ref.gate_proj(h, w, b, ops.GATE_CAP_TANH, ops.GATE_LOGSIG_CAP_TANH, N // 2, 9.0)
    got = ops.gate_proj(h.to(gpu), w.to(gpu), b.to(gpu), ops.GATE_CAP_TANH,
                        ops.GATE_LOGSIG_CAP_TANH, N // 2, 9.0)
    torch.testing.assert_close(got.cpu(), want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("dt", DT)
def test_window_attention_many_decode_rows(gpu, dt):
    """A decode batch large enough (rows x kv heads >= 512) for the 4-wave workgroups."""
    torch.manual_seed(8)
    H, G, dk, dv, bs, window, keep = 4, 2, 64, 32, 8, 50, 3
    g = torch.Generator().manual_seed(9)
    D_ctx = torch.randint(1, 200, (300,), generator=g).tolist()
    mb = max(D_ctx) // bs + 1
    nb = 64
    tables = torch.randint(1, nb, (len(D_ctx), mb), generator=g).to(torch.int32)
    kc = (torch.randn(nb, G, bs, dk) * 0.7).to(dt)
    vc = torch.randn(nb, G, bs, dv).to(dt)
    m = _meta([], [], D_ctx, tables)
    q = torch.randn(len(D_ctx), H, dk).to(dt)
    pos = torch.tensor([c - 1 for c in D_ctx])
    want = ops.window_attention(q, kc, vc, pos, m, 0.2, window, keep, None)
    got = ops.window_attention(q.to(gpu), kc.to(gpu), vc.to(gpu), pos.to(gpu), _to(m, gpu), 0.2,
                               window, keep, None)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dt))
