"""Each mechanism of the Konovik decoder alone (the product's op or mixer module) against
the numpy oracle's function for it, on the CPU reference ops and, with ``-m gpu``, on the
HIP kernels.  The visibility tests plant ONE key whose score dwarfs all others, so a key
that is wrongly seen or wrongly hidden flips the output between "its value" and "not"."""
import types

import numpy as np
import pytest
import torch

import konovik_oracle as oracle
from kubernetes_gpu_cluster_amd import ops
from kubernetes_gpu_cluster_amd.models.attention import ForwardContext, LatentAttention
from kubernetes_gpu_cluster_amd.models.configs import (FeedForwardSpec, MixerSpec, RotarySpec,
                                                       WindowSpec)
from kubernetes_gpu_cluster_amd.models.moe import SigmoidRoutedExperts
from kubernetes_gpu_cluster_amd.models.recurrent import MinGRUMixer
from kubernetes_gpu_cluster_amd.parallel.state import get_state

DEV = [pytest.param("cpu", id="cpu"), pytest.param("cuda", marks=pytest.mark.gpu, id="gpu")]


def dev_of(name):
    if name == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device(name)


def f32(a, dev):
    return torch.tensor(np.asarray(a), dtype=torch.float32, device=dev)


def meta_for(chunks, decodes, tables, dev, slots=None):
    """chunks: [(first position, length)], decodes: [position] -> (metadata, positions)."""
    m = types.SimpleNamespace()
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)   # noqa: E731
    P, D = len(chunks), len(decodes)
    qsl = np.concatenate([[0], np.cumsum([n for _, n in chunks])]).astype(int).tolist()
    m.num_prefills, m.num_decodes, m.num_prefill_tokens = P, D, qsl[-1]
    m.query_start_loc = i32(qsl) if P else None
    m.prefill_seq_lens = i32([a + n for a, n in chunks]) if P else None
    m.prefill_block_tables = tables[:P].contiguous().to(dev) if P and tables is not None else None
    m.decode_ctx_lens = i32([p + 1 for p in decodes]) if D else None
    m.decode_block_tables = tables[P:P + D].contiguous().to(dev) if D and tables is not None else None
    m.state_slots = i32(slots) if slots is not None else None
    pos = [p for a, n in chunks for p in range(a, a + n)] + list(decodes)
    return m, torch.tensor(pos, dtype=torch.int64, device=dev)


def steps_of(n, cuts):
    """[(lo, hi, is a decode row)] for a sequence fed in portions `cuts` (the last repeats)."""
    out, lo, i = [], 0, 0
    while lo < n:
        c = cuts[min(i, len(cuts) - 1)]
        i += 1
        hi = min(n, lo + c)
        out.append((lo, hi, hi - lo == 1 and lo > 0))
        lo = hi
    return out


# ---------------------------------------------------------------- norms, shift, small ops
@pytest.mark.parametrize("dev", DEV)
def test_residual_norm(dev):
    dev = dev_of(dev)
    rng = np.random.default_rng(0)
    x, y = rng.normal(size=(5, 70)) * 3, rng.normal(size=(5, 70))
    w, wn = rng.normal(size=70), rng.normal(size=70)
    xs = f32(x, dev)
    h = ops.residual_norm(xs, f32(y, dev), 0.3, f32(w, dev), 1e-3, torch.float32)
    np.testing.assert_allclose(xs.cpu().numpy(), x + 0.3 * y, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(h.cpu().numpy(), oracle.rms(x + 0.3 * y, 1e-3) * w, rtol=3e-5, atol=3e-5)
    # a normed addend; no output; then the plain copy and the in-place norm
    xs = f32(x, dev)
    assert ops.residual_norm(xs, f32(y, dev), 0.5, None, 1e-3, None, add_norm_w=f32(wn, dev)) is None
    want = x + 0.5 * oracle.rms(y, 1e-3) * wn
    np.testing.assert_allclose(xs.cpu().numpy(), want, rtol=3e-5, atol=3e-5)
    c = ops.residual_norm(xs, None, 1.0, None, 1e-3, torch.float32)
    np.testing.assert_allclose(c.cpu().numpy(), want, rtol=3e-5, atol=3e-5)
    ops.residual_norm(xs, None, 1.0, f32(w, dev), 1e-3, torch.float32, out=xs)
    np.testing.assert_allclose(xs.cpu().numpy(), oracle.rms(want, 1e-3) * w, rtol=5e-5, atol=5e-5)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("cuts", [[23], [2], [7, 1], [1], [3, 9, 1, 1, 6]])
def test_token_shift_over_steps(dev, cuts):
    """Portions, decode rows and a second sequence in the same steps; slot 2 held another
    sequence's row before."""
    dev = dev_of(dev)
    rng = np.random.default_rng(1)
    n, W = 23, 37
    h, h2, mu = rng.normal(size=(n, W)), rng.normal(size=(n, W)), rng.uniform(size=W)
    state = torch.full((4, W), 7.0, device=dev)
    got, got2 = [], []
    for lo, hi, dec in steps_of(n, cuts):
        # the other sequence always decodes one token per step, from position 0 on
        t2 = len(got2)
        first2 = t2 == 0
        chunks = ([] if dec else [(lo, hi - lo)]) + ([(0, 1)] if first2 else [])
        decs = ([lo] if dec else []) + ([] if first2 else [t2])
        rows = ([] if dec else [h[lo:hi]]) + ([h2[:1]] if first2 else []) + \
               ([h[lo:hi]] if dec else []) + ([] if first2 else [h2[t2:t2 + 1]])
        slots = ([] if dec else [2]) + ([0] if first2 else []) + ([2] if dec else []) + \
                ([] if first2 else [0])
        m, _ = meta_for(chunks, decs, None, dev, slots)
        out = ops.token_shift(f32(np.concatenate(rows), dev), f32(mu, dev), state, m,
                              torch.float32).cpu().numpy()
        if dec:
            got2.append(out[:1] if first2 else out[-1:])
            got.append(out[1:2] if first2 else out[:1])
        else:
            got.append(out[:hi - lo])
            got2.append(out[hi - lo:hi - lo + 1])
    np.testing.assert_allclose(np.concatenate(got), oracle.token_shift(h, mu), rtol=1e-5, atol=1e-5)
    k = len(got2)
    np.testing.assert_allclose(np.concatenate(got2), oracle.token_shift(h2[:k], mu), rtol=1e-5,
                               atol=1e-5)


@pytest.mark.parametrize("dev", DEV)
def test_yarn_table_and_side_gate(dev):
    dev = dev_of(dev)
    for dims, base, yarn in ((8, 100.0, (3.0, 16.0, 4.0, 1.0)), (16, 5000.0, (8.0, 1024.0, 16.0, 2.0)),
                             (6, 50.0, None)):
        sc = dict(zip(("factor", "original", "fast", "slow"), yarn)) if yarn else None
        f, mag = oracle.yarn_frequencies(dims, base, sc)
        tab = ops.ref.rope_table_yarn(dims, 50, base, yarn).numpy()
        ang = np.arange(50)[:, None] * f[None]
        np.testing.assert_allclose(tab, np.concatenate([np.cos(ang) * mag, np.sin(ang) * mag], -1),
                                   rtol=2e-4, atol=2e-4)
    rng = np.random.default_rng(2)
    pre, table = rng.normal(size=(9, 5)) * 2, rng.normal(size=(30, 20))
    ids = rng.integers(0, 30, 9)
    got = ops.side_gate(f32(pre, dev), torch.tensor(ids, device=dev), f32(table, dev), 10)
    np.testing.assert_allclose(got.cpu().numpy(), oracle.gelu_tanh(pre) * table[ids, 10:15],
                               rtol=2e-5, atol=2e-5)
    z = rng.normal(size=(4, 33))
    np.testing.assert_allclose(ops.relu_sq(f32(z, dev)).cpu().numpy(), np.maximum(z, 0) ** 2,
                               rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dev,dtype", [pytest.param("cpu", torch.float32, id="cpu"),
                                       pytest.param("cuda", torch.float32, marks=pytest.mark.gpu, id="gpu-fp32"),
                                       pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu, id="gpu-bf16")])
@pytest.mark.parametrize("rows", [3, 300])
def test_side_input_end_of_layer(dev, dtype, rows):
    """x += m y; the gated side projection, RMS-normed, joins x; then the next norm.  Few
    rows of 16-bit activations take the one-kernel path on the GPU, many rows the GEMMs."""
    dev = dev_of(dev)
    rng = np.random.default_rng(12)
    W, n, vocab, layer = 72, 8, 40, 2
    rnd = lambda *sh: torch.tensor(rng.normal(size=sh), dtype=torch.float32).to(dtype)   # noqa: E731
    x = torch.tensor(rng.normal(size=(rows, W)) * 2, dtype=torch.float32)
    y, wg, wp, table = rnd(rows, W), rnd(n, W) / 6, rnd(W, n), rnd(vocab, 4 * n)
    sw, nw = rng.normal(size=W) + 1, rng.normal(size=W) + 1
    ids = rng.integers(0, vocab, rows)
    xs = x.clone().to(dev)
    h = ops.side_input(xs, y.to(dev), 0.4, wg.to(dev), wp.to(dev), torch.tensor(ids, device=dev),
                       table.to(dev), layer * n, f32(sw, dev), f32(nw, dev), 1e-5, torch.float32)
    d = lambda t: t.float().double().numpy()   # noqa: E731
    x1 = x.double().numpy() + 0.4 * d(y)
    wts = {"side.embed": d(table), "side.gate": d(wg), "side.proj": d(wp), "side.norm": sw}
    x2 = x1 + 0.4 * oracle.side_input(x1, ids, wts, "", layer, n, 1e-5)
    tol = 3e-4 if dtype == torch.float32 else 4e-2
    np.testing.assert_allclose(xs.cpu().numpy(), x2, rtol=tol, atol=tol)
    np.testing.assert_allclose(h.cpu().numpy(), oracle.rms(x2, 1e-5) * nw, rtol=tol, atol=tol)
    # without a next norm: the stream only
    xs = x.clone().to(dev)
    assert ops.side_input(xs, y.to(dev), 0.4, wg.to(dev), wp.to(dev), torch.tensor(ids, device=dev),
                          table.to(dev), layer * n, f32(sw, dev), None, 1e-5, None) is None
    np.testing.assert_allclose(xs.cpu().numpy(), x2, rtol=tol, atol=tol)


# ---------------------------------------------------------------- minGRU
def _mingru_case(dev, width, hidden, n, cuts, seed):
    get_state()
    torch.manual_seed(seed)
    spec = MixerSpec("mingru", 1, width, width, width=width)
    mod = MinGRUMixer(hidden, spec, torch.float32, dev)
    for p in mod.parameters():
        p.data.copy_(torch.randn(p.shape) * 1.5 / p.shape[-1] ** 0.5)
    h = torch.randn(n, hidden)
    state = torch.full((3, width), -5.0, device=dev)      # stale: the slot was used before
    outs = []
    for lo, hi, dec in steps_of(n, cuts):
        m, pos = meta_for([] if dec else [(lo, hi - lo)], [lo] if dec else [], None, dev, [1])
        outs.append(mod(h[lo:hi].to(dev), pos, ForwardContext(m, []), state).cpu())
    sd = {k: v.detach().cpu().double().numpy() for k, v in mod.state_dict().items()}
    w = sd["zxg_proj.weight"]
    wts = {"mix.z": w[:width], "mix.x": w[width:2 * width], "mix.g": w[2 * width:],
           "mix.z.b": sd["zx_bias"][:width], "mix.x.b": sd["zx_bias"][width:],
           "mix.o": sd["o_proj.weight"]}
    return torch.cat(outs).numpy(), oracle.mingru(h.double().numpy(), wts, "", {"width": width})


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("cuts", [[50], [2], [17, 1], [1], [9, 8, 1, 1, 20]])
def test_mingru_alone(dev, cuts):
    dev = dev_of(dev)
    got, want = _mingru_case(dev, 70, 24, 50, cuts, 3)
    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("dev", DEV)
def test_mingru_long_chunks(dev):
    """Chunks long enough for the block-parallel scan (blocks of 64 tokens, a ragged last
    block), continued from and handing over to the token-order scan."""
    dev = dev_of(dev)
    got, want = _mingru_case(dev, 70, 24, 1300, [3, 650, 1, 1, 577, 20, 1], 11)
    np.testing.assert_allclose(got, want, rtol=3e-4, atol=3e-4)


@pytest.mark.parametrize("dev", DEV)
def test_mingru_scan_long_chunk_beside_decode_rows(dev):
    """One step holds two long chunks (one from position 0, one continuing a state) and two
    decode rows of other sequences; plain numpy recurrences are the expectation."""
    dev = dev_of(dev)
    rng = np.random.default_rng(13)
    n, lens = 70, [700, 530]
    T = sum(lens) + 2
    zxg, bias = rng.normal(size=(T, 3 * n)), rng.normal(size=2 * n) * 0.5
    state = rng.normal(size=(5, n))
    m, _ = meta_for([(0, lens[0]), (40, lens[1])], [9, 0], None, dev, [3, 1, 0, 4])
    st = f32(state, dev)
    got = ops.mingru_scan(f32(zxg, dev), f32(bias, dev), st, m, n, torch.float32).cpu().numpy()
    z = oracle.sigmoid(zxg[:, :n] + bias[:n])
    u = zxg[:, n:2 * n] + bias[n:]
    cand = np.where(u >= 0, u + 0.5, oracle.sigmoid(u))
    gate = oracle.silu(zxg[:, 2 * n:])
    want, end = np.zeros((T, n)), {}
    for a, ln, s0, slot in ((0, 700, None, 3), (700, 530, state[1], 1), (1230, 1, state[0], 0),
                            (1231, 1, None, 4)):
        S = np.zeros(n) if s0 is None else s0.copy()
        for t in range(a, a + ln):
            S = (1 - z[t]) * S + z[t] * cand[t]
            want[t] = S * gate[t]
        end[slot] = S
    np.testing.assert_allclose(got, want, rtol=3e-4, atol=3e-4)
    for slot, S in end.items():
        np.testing.assert_allclose(st[slot].cpu().numpy(), S, rtol=3e-4, atol=3e-4)
    np.testing.assert_allclose(st[2].cpu().numpy(), state[2], rtol=1e-6)      # untouched


# ---------------------------------------------------------------- latent attention
def _latent_case(dev, spec, hidden, h, cuts, page, seed, eps=1e-5, prepare=None):
    """Run the LatentAttention module over a sequence cut into steps -> ([n, hidden], oracle)."""
    get_state()
    torch.manual_seed(seed)
    n = h.shape[0]
    mod = LatentAttention(hidden, spec, eps, torch.float32, dev)
    for name, p in mod.named_parameters():
        p.data.copy_(torch.randn(p.shape) * 1.5 / p.shape[-1] ** 0.5 + (1.0 if "norm" in name else 0))
    if prepare is not None:
        prepare(mod)
    mod.prepare({}, n + 1, dev)
    pages = -(-n // page)
    table = (torch.randperm(pages) + 1).to(torch.int32)[None]
    cache = torch.zeros(pages + 1, 1, page, spec.kv_rank + spec.rot_dims, device=dev)
    empty = torch.zeros(pages + 1, 1, page, 0, device=dev)
    outs = []
    for lo, hi, dec in steps_of(n, cuts):
        m, pos = meta_for([] if dec else [(lo, hi - lo)], [lo] if dec else [], table, dev)
        m.slot_mapping = (table[0].long()[pos.cpu() // page] * page + pos.cpu() % page).to(dev)
        outs.append(mod(h[lo:hi].to(dev), pos, ForwardContext(m, [(cache, empty)]), 0).cpu())
    sd = {k: v.detach().cpu().double().numpy() for k, v in mod.state_dict().items()}
    H, d, r, dv, rank = spec.heads, spec.dim, spec.rot_dims, spec.vdim, spec.kv_rank
    w = sd["proj.weight"]
    wts = {"mix.q": w[: mod.n_q], "mix.dkv": w[mod.n_q: mod.n_q + mod.n_kv],
           "mix.g": w[mod.n_q + mod.n_kv:], "mix.dkv.norm": sd["norm_weight"],
           "mix.uk": sd["w_uk"].reshape(H * d, rank),
           "mix.uv": sd["w_uv"].transpose(0, 2, 1).reshape(H * dv, rank), "mix.o": sd["o_proj.weight"]}
    cfgm = {"heads": H, "dim": d, "rot_dim": r, "vdim": dv, "kv_rank": rank, "scale": spec.scale}
    if spec.window:
        cfgm["mask"] = {"size": spec.window.size}
    if r:
        rs = spec.rotary
        cfgm["rot"] = {"dims": r, "base": rs.base}
        if rs.yarn:
            cfgm["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), rs.yarn))
    return torch.cat(outs).numpy(), oracle.latent_attention(h.double().numpy(), wts, "", cfgm, eps), wts, cfgm


def latent_spec(heads=5, dim=12, rot=6, vdim=10, rank=20, size=9, scale=0.4, yarn=(3.0, 16.0, 4.0, 1.0)):
    return MixerSpec("latent_attention", heads, dim, vdim, kv_heads=1, scale=scale, rot_dims=rot,
                     window=WindowSpec(size) if size else None, kv_rank=rank,
                     rotary=RotarySpec(rot, 50.0, True, yarn) if rot else None)


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("cuts", [[40], [13, 1], [2], [5, 9, 1, 1, 7]])
def test_latent_attention_alone(dev, cuts):
    dev = dev_of(dev)
    torch.manual_seed(5)
    got, want, _, _ = _latent_case(dev, latent_spec(), 28, torch.randn(40, 28), cuts, 8, 4)
    np.testing.assert_allclose(got, want, rtol=3e-4, atol=3e-4)
    # one head, no window, rotary part only half of the table's use, no scaling
    got, want, _, _ = _latent_case(dev, latent_spec(1, 8, 8, 8, 8, 0, 0.5, None), 16,
                                   torch.randn(40, 16), cuts, 8, 6)
    np.testing.assert_allclose(got, want, rtol=3e-4, atol=3e-4)


def _planted(dev, size, far, decode, n=330):
    """Hidden channel 0 is read only by one rotary key column, channel 1 only by the same
    rotary column of every head's query, both with a large gain; token j = n - 1 - far alone
    carries channel 0 and the last token alone channel 1, so score (last, j) ~ gain^2 dwarfs
    all others wherever j is visible.  The column belongs to a pair that barely turns over
    the distance (a huge base).  -> (module output of the last row, oracle's last row)."""
    spec = MixerSpec("latent_attention", 2, 8, 6, kv_heads=1, scale=1.0, rot_dims=4,
                     window=WindowSpec(size) if size else None, kv_rank=12,
                     rotary=RotarySpec(4, 1e9, True, None))
    torch.manual_seed(7)
    h = torch.randn(n, 20) * 0.5
    h[:, :2] = 0.0
    h[n - 1 - far, 0] = 1.0
    h[n - 1, 1] = 1.0

    def plant(mod):
        w = mod.proj.weight.data
        w[:, :2] = 0.0
        for head in range(spec.heads):
            w[head * (spec.dim + 4) + spec.dim + 2, 1] = 9.0
        w[mod.n_q + spec.kv_rank + 2, 0] = 9.0
    got, want, _, _ = _latent_case(dev, spec, 20, h, [n - 1, 1] if decode else [n], 16, 8,
                                   prepare=plant)
    return got, want


@pytest.mark.parametrize("dev", DEV)
@pytest.mark.parametrize("decode", [False, True])
def test_planted_key_at_window_edges(dev, decode):
    """The planted key sits just inside and just outside every window, at page borders (16)
    and key-tile borders (64), and hundreds of tokens back; the last token is a prompt row
    or a decode row.  Inside the window the last row is the planted token's value, outside
    it is not: the two oracle rows differ by far more than the tolerance."""
    dev = dev_of(dev)
    for size, fars in ((9, (8, 9)), (64, (63, 64)), (65, (64, 65)), (16, (15, 16)), (0, (300, 17))):
        rows = []
        for far in fars:
            got, want = _planted(dev, size, far, decode)
            np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3)
            rows.append(want[-1])
        if size:
            assert np.abs(rows[0] - rows[1]).max() > 0.1      # seen vs hidden shows


# ---------------------------------------------------------------- routed experts
def _experts_case(dev, spec, hidden, n, seed, dtype=torch.float32, spread=3.0):
    get_state()
    torch.manual_seed(seed)
    mod = SigmoidRoutedExperts(hidden, spec, dtype, dev)
    for name, p in mod.named_parameters():
        g = spread if name == "gates" else 1.5
        p.data.copy_((torch.randn(p.shape) * g / p.shape[-1] ** 0.5).to(p.dtype))
    mod.correction.data.copy_(torch.randn(spec.experts) * 0.3)
    h = torch.randn(n, hidden).to(dtype)
    got = mod(h.to(dev)).float().cpu().numpy()
    sd = {k: v.detach().float().cpu().double().numpy() for k, v in mod.state_dict().items()}
    wts = {"mlp.router": sd["gates"][: spec.experts], "mlp.correction": sd["correction"]}
    for e in range(spec.experts):
        wts["mlp.e%d.up" % e], wts["mlp.e%d.down" % e] = sd["w_up"][e], sd["w_down"][e]
    mlp = {"kind": "moe", "router": {"experts": spec.experts, "top": spec.top, "scale": spec.route_scale}}
    if spec.shared_ff:
        mlp["shared"] = {"ff": spec.shared_ff}
        wts["mlp.shared.up"], wts["mlp.shared.down"] = sd["shared_up.weight"], sd["shared_down.weight"]
        wts["mlp.shared.sg"] = sd["gates"][spec.experts:]
    margins = []
    want = oracle.feed_forward(h.float().double().numpy(), wts, "", mlp, margins)
    firm = margins[0] > (1e-4 if dtype == torch.float32 else 0.03) if margins else np.ones(n, bool)
    return mod, got, want, firm


@pytest.mark.parametrize("dev", DEV)
def test_routed_experts_alone(dev):
    dev = dev_of(dev)
    for spec in (FeedForwardSpec("moe", 24, "relu2", 7, 3, 1.7, 20),
                 FeedForwardSpec("moe", 16, "relu2", 2, 1, 1.0, 0),
                 FeedForwardSpec("moe", 8, "relu2", 70, 5, 0.5, 8),
                 FeedForwardSpec("moe", 8, "relu2", 4, 4, 2.0, 0)):
        _, got, want, firm = _experts_case(dev, spec, 40, 33, 9)
        assert firm.sum() >= 30
        np.testing.assert_allclose(got[firm], want[firm], rtol=3e-4, atol=3e-4)


@pytest.mark.gpu
def test_routed_experts_grouped_gemm():
    """Shapes the grouped matrix-core GEMM takes (16-bit activations), decode-size and
    prefill-size batches, against the oracle on the same bf16 weights."""
    dev = dev_of("cuda")
    spec = FeedForwardSpec("moe", 128, "relu2", 8, 2, 1.5, 128)
    for n in (3, 70, 600):
        mod, got, want, firm = _experts_case(dev, spec, 256, n, 10, torch.bfloat16)
        assert mod.native
        scale = np.abs(want).max()
        assert np.abs(got[firm] - want[firm]).max() < 0.03 * scale


def test_route_choice_uses_the_correction_but_weights_do_not():
    scores = torch.tensor([[0.9, 0.5, 0.4, 0.1]])
    corr = torch.tensor([-0.6, 0.0, 0.0, 0.25])
    w, ids = ops.moe_route_sigmoid(scores, corr, 2, 2.0)
    assert sorted(ids[0].tolist()) == [1, 2]
    got = dict(zip(ids[0].tolist(), w[0].tolist()))
    assert abs(got[1] - 2.0 * 0.5 / 0.9) < 1e-6 and abs(got[2] - 2.0 * 0.4 / 0.9) < 1e-6
