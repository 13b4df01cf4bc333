"""Each mechanism of the hybrid decoders alone (the product's op or mixer module) against
the numpy oracle's function for it, on the CPU reference ops and, with ``-m gpu``, on the
HIP kernels.  The visibility test plants ONE key whose score dwarfs all others, so a key
that is wrongly seen or wrongly hidden flips the output between "its value" and "not"."""
import types

import numpy as np
import pytest
import torch

import dilavik_oracle as oracle
from kubernetes_gpu_cluster_amd import ops
from kubernetes_gpu_cluster_amd.models.attention import ForwardContext, WindowedAttention
from kubernetes_gpu_cluster_amd.models.configs import MixerSpec, WindowSpec
from kubernetes_gpu_cluster_amd.models.recurrent import MLSTMMixer
from kubernetes_gpu_cluster_amd.parallel.state import get_state

DEV = [pytest.param("cpu", id="cpu"), pytest.param("cuda", marks=pytest.mark.gpu, id="gpu")]


def dev_of(name):
    if name == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device(name)


def meta_for(chunks, decodes, tables, dev, slots=None):
    """chunks: [(first position, length)], decodes: [position] -> (metadata, positions)."""
    m = types.SimpleNamespace()
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)   # noqa: E731
    P, D = len(chunks), len(decodes)
    qsl = np.concatenate([[0], np.cumsum([n for _, n in chunks])]).astype(int).tolist()
    m.num_prefills, m.num_decodes, m.num_prefill_tokens = P, D, qsl[-1]
    m.query_start_loc = i32(qsl) if P else None
    m.prefill_seq_lens = i32([a + n for a, n in chunks]) if P else None
    m.prefill_block_tables = tables[:P].contiguous().to(dev) if P else None
    m.decode_ctx_lens = i32([p + 1 for p in decodes]) if D else None
    m.decode_block_tables = tables[P:P + D].contiguous().to(dev) if D else None
    m.state_slots = i32(slots) if slots is not None else None
    pos = [p for a, n in chunks for p in range(a, a + n)] + list(decodes)
    return m, torch.tensor(pos, dtype=torch.int64, device=dev)


@pytest.mark.parametrize("dev", DEV)
def test_group_norm_xielu_depth_average(dev):
    dev = dev_of(dev)
    rng = np.random.default_rng(0)
    x = rng.normal(size=(5, 60)) * 4
    w = rng.normal(size=60)
    for groups in (1, 3, 5):
        got = ops.group_rms_norm(torch.tensor(x, dtype=torch.float32, device=dev),
                                 torch.tensor(w, dtype=torch.float32, device=dev), groups, 1e-3,
                                 torch.float32)
        np.testing.assert_allclose(got.cpu().numpy(), oracle.group_norm(x, w, groups, 1e-3),
                                   rtol=2e-5, atol=2e-5)
    z = rng.normal(size=(4, 33)) * 3
    p, q = 0.4, -1.1
    ab = torch.tensor([oracle.softplus(p), 0.5 + oracle.softplus(q)], dtype=torch.float32, device=dev)
    got = ops.xielu(torch.tensor(z, dtype=torch.float32, device=dev), ab)
    np.testing.assert_allclose(got.cpu().numpy(), oracle.xielu(z, p, q), rtol=2e-5, atol=2e-5)
    # end of layer 2 of a depth-averaged stack: results X_0..X_2 known, X_3 = x + y
    res = [rng.normal(size=(5, 60)) for _ in range(3)]
    y = rng.normal(size=(5, 60))
    coef = rng.normal(size=4)
    hist = torch.zeros(6, 8, 60, device=dev)
    for j, r in enumerate(res):
        hist[j, :5] = torch.tensor(r, dtype=torch.float32)
    xs = torch.tensor(x, dtype=torch.float32, device=dev)
    h = ops.depth_mix_norm(xs, hist, 2, torch.tensor(y, dtype=torch.float32, device=dev),
                           torch.tensor(coef, dtype=torch.float32, device=dev),
                           torch.tensor(w, dtype=torch.float32, device=dev), 3, 1e-3, torch.float32)
    want = oracle.depth_average(res + [x + y], coef)
    np.testing.assert_allclose(xs.cpu().numpy(), want, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(hist[3, :5].cpu().numpy(), x + y, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(h.cpu().numpy(), oracle.group_norm(want, w, 3, 1e-3), rtol=5e-5,
                               atol=5e-5)


def _attention_case(dev, spec, hidden, n, cuts, page, seed):
    """Run the WindowedAttention module over a sequence cut into steps (sizes `cuts`, the
    last repeating; a one-token step after the first is a decode row) -> [n, hidden]."""
    get_state()
    torch.manual_seed(seed)
    mod = WindowedAttention(hidden, spec, 0, torch.float32, dev)
    for p in mod.parameters():
        p.data.copy_(torch.randn(p.shape) * 1.5 / p.shape[-1] ** 0.5)
    mod.prepare({}, n + 1, dev)
    h = torch.randn(n, hidden)
    pages = -(-n // page)
    table = (torch.randperm(pages) + 1).to(torch.int32)[None]
    kc = torch.zeros(pages + 1, spec.kv_heads, page, spec.dim, device=dev)
    vc = torch.zeros(pages + 1, spec.kv_heads, page, spec.vdim, device=dev)
    outs, lo, i = [], 0, 0
    while lo < n:
        c = cuts[min(i, len(cuts) - 1)]
        i += 1
        hi = min(n, lo + c)
        dec = hi - lo == 1 and lo > 0
        m, pos = meta_for([] if dec else [(lo, hi - lo)], [lo] if dec else [], table, dev)
        m.slot_mapping = (table[0].long()[pos.cpu() // page] * page + pos.cpu() % page).to(dev)
        ctx = ForwardContext(m, [(kc, vc)])
        outs.append(mod(h[lo:hi].to(dev), pos, ctx).cpu())
        lo = hi
    sd = {k: v.detach().cpu().double().numpy() for k, v in mod.state_dict().items()}
    H, G, dk = spec.heads, spec.kv_heads, spec.dim
    wq = sd["qkv_proj.weight"]
    wts = {"mix.q": wq[: H * dk], "mix.k": wq[H * dk:(H + G) * dk], "mix.v": wq[(H + G) * dk:],
           "mix.g": sd["gate"], "mix.o": sd["o_proj.weight"]}
    cfgm = {"heads": H, "kv_heads": G, "dim": dk, "vdim": spec.vdim, "scale": spec.scale,
            "rot": {"dims": spec.rot_dims, "base": spec.rot_base},
            "mask": {"size": spec.window.size, "keep_first": spec.window.keep_first}}
    want = oracle.attention_mixer(h.double().numpy(), wts, "", cfgm)
    return torch.cat(outs).numpy(), want


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("cuts", [[40], [13, 1], [2], [5, 9, 1, 1, 7]])
def test_attention_mixer_alone(dev, cuts):
    dev = dev_of(dev)
    spec = MixerSpec("attention", 6, 20, 12, kv_heads=3, scale=0.4, rot_dims=8, rot_base=50.0,
                     window=WindowSpec(6, 2), head_gate=True)
    got, want = _attention_case(dev, spec, 48, 40, cuts, 4, 1)
    np.testing.assert_allclose(got, want, rtol=3e-4, atol=3e-4)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("decode", [False, True])
def test_visibility_with_a_standout_key(dev, decode):
    """Query i (a prompt row, or a decode row) and key j share a direction scaled so that
    softmax puts all weight on j whenever j is visible: the output is then v_j.  Pairs sit
    just inside / outside the window, on the kept first tokens and the next ones, on page
    borders, and hundreds of tokens back."""
    dev = dev_of(dev)
    page, n, size, keep = 16, 400, 300, 3
    dk, dv = 8, 8
    pairs = [(i, j) for i in (399, 352, 320, 303, 302, 64, 17, 16, 5, 2, 0)
             for j in (i, i - 1, i - size + 1, i - size, i - size - 1, 0, keep - 1, keep, keep + 1,
                       15, 16, 17, i - 100, i - 299) if 0 <= j <= i]
    rng = torch.Generator().manual_seed(3)
    k = torch.randn(n, 1, dk, generator=rng) * 0.1
    v = torch.randn(n, 1, dv, generator=rng)
    pages = n // page
    table = (torch.randperm(pages, generator=rng) + 1).to(torch.int32)[None]
    for i, j in pairs:
        kk = k.clone()
        kk[j, 0] = 0
        kk[j, 0, 0] = 40.0
        q = torch.zeros(1, 1, dk)
        q[0, 0, 0] = 40.0
        kc = torch.zeros(pages + 1, 1, page, dk)
        vc = torch.zeros(pages + 1, 1, page, dv)
        idx = torch.arange(n)
        kc[table[0].long()[idx // page], :, idx % page] = kk
        vc[table[0].long()[idx // page], :, idx % page] = v
        if decode:
            m, pos = meta_for([], [i], table, dev)
        else:
            m, pos = meta_for([(i, 1)] if i == 0 else [(i - 1, 2)], [], table, dev)
            q = torch.cat([torch.zeros(1, 1, dk), q]) if i else q
        out = ops.window_attention(q.to(dev), kc.to(dev), vc.to(dev), pos, m, 1.0, size, keep, None)
        out = out[-1].cpu()
        hit = bool(torch.allclose(out, v[j, 0], atol=1e-3))
        assert hit == oracle.visible(i, j, size, keep), (i, j, decode)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("cuts", [[37], [12, 1], [2], [3, 8, 1, 1, 16]])
def test_mlstm_mixer_alone(dev, cuts):
    """The MLSTMMixer module over a sequence cut into steps (state carried in its slot,
    which first holds another sequence's state) against the oracle's recurrence."""
    dev = dev_of(dev)
    get_state()
    spec = MixerSpec("mlstm", 3, 10, 14, gate_cap=6.0)
    hidden, n, eps = 40, 37, 1e-4
    torch.manual_seed(5)
    mod = MLSTMMixer(hidden, spec, 0, eps, torch.float32, dev)
    for name, p in mod.named_parameters():
        gain = 4.0 if name == "if_weight" else 1.5
        p.data.copy_(torch.randn(p.shape) * (gain / p.shape[-1] ** 0.5 if p.dim() == 2 else 1.0))
    H, d, dv = spec.heads, spec.dim, spec.vdim
    states = [(torch.randn(3, H, d, dv, device=dev), torch.randn(3, H, d, device=dev),
               torch.rand(3, H, device=dev))]              # stale contents of the slots
    h = torch.randn(n, hidden)
    outs, lo, i = [], 0, 0
    while lo < n:
        c = cuts[min(i, len(cuts) - 1)]
        i += 1
        hi = min(n, lo + c)
        dec = hi - lo == 1 and lo > 0
        m, pos = meta_for([] if dec else [(lo, hi - lo)], [lo] if dec else [],
                          torch.zeros(1, 1, dtype=torch.int32), dev, slots=[2])
        ctx = ForwardContext(m, [], states=states)
        outs.append(mod(h[lo:hi].to(dev), pos, ctx).cpu())
        lo = hi
    sd = {k: v.detach().cpu().double().numpy() for k, v in mod.state_dict().items()}
    wq = sd["qkvg_proj.weight"]
    wts = {"mix.q": wq[: H * d], "mix.k": wq[H * d: 2 * H * d],
           "mix.v": wq[2 * H * d: 2 * H * d + H * dv], "mix.g": wq[2 * H * d + H * dv:],
           "mix.i": sd["if_weight"][:H], "mix.f": sd["if_weight"][H:],
           "mix.i.b": sd["if_bias"][:H], "mix.f.b": sd["if_bias"][H:],
           "mix.norm": sd["norm_weight"], "mix.o": sd["o_proj.weight"]}
    want = oracle.mlstm_mixer(h.double().numpy(), wts, "",
                              {"heads": H, "dim": d, "vdim": dv, "gate_cap": 6.0}, eps)
    np.testing.assert_allclose(torch.cat(outs).numpy(), want, rtol=5e-4, atol=5e-4)


@pytest.mark.parametrize("dev", DEV)
def test_rotary_pairs_and_partial_dims(dev):
    dev = dev_of(dev)
    H, G, dk, dv, rot, n = 2, 1, 10, 4, 6, 9
    torch.manual_seed(7)
    qkv = torch.randn(n, (H + G) * dk + G * dv)
    table = ops.ref.rope_table(rot, 64, 30.0).to(dev)
    pos = torch.tensor([0, 1, 2, 3, 4, 5, 6, 7, 8], dtype=torch.int64)
    kc = torch.zeros(4, G, 4, dk, device=dev)
    vc = torch.zeros(4, G, 4, dv, device=dev)
    slots = torch.tensor([4, 5, 6, 7, 8, 9, 10, -1, 12], dtype=torch.int64)
    q = ops.rope_kv_store(qkv.to(dev), pos.to(dev), table, kc, vc, slots.to(dev), H, G, dk, dv)
    want_q = oracle.rotate(qkv[:, : H * dk].double().numpy().reshape(n, H, dk), rot, 30.0)
    want_k = oracle.rotate(qkv[:, H * dk:(H + G) * dk].double().numpy().reshape(n, G, dk), rot, 30.0)
    np.testing.assert_allclose(q.cpu().numpy(), want_q, rtol=1e-5, atol=1e-5)
    kflat = kc.cpu().numpy().transpose(0, 2, 1, 3).reshape(16, G, dk)
    np.testing.assert_allclose(kflat[4:11], want_k[:7], rtol=1e-5, atol=1e-5)
    assert np.all(kflat[11] == 0)                     # slot -1: nothing written
    np.testing.assert_allclose(kflat[12], want_k[8], rtol=1e-5, atol=1e-5)
    vflat = vc.cpu().numpy().transpose(0, 2, 1, 3).reshape(16, G, dv)
    np.testing.assert_array_equal(vflat[12], qkv[8, (H + G) * dk:].numpy().reshape(G, dv))
