"""HIP kernels of the layer-norm stream ops, query/key norm, any-shape
attention and the recurrences against the plain-PyTorch reference ops (f32
upcast), on sizes that hit vector and scalar paths, state reuse and padding
rows."""

import pytest
import torch

from vllm_tgis_adapter_amd import ops
from vllm_tgis_adapter_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _close(a, b, dtype, what=""):
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    a, b = a.float().cpu(), b.float().cpu()
    assert a.shape == b.shape, what
    if a.numel() == 0:
        return
    scale = max(1.0, float(b.abs().max()))
    err = float((a - b).abs().max()) / scale
    assert err < tol, f"{what}: {err}"


def _seqs(spec):
    """spec: [(new rows, total length, slot)] -> loc, lens, slots (int32 cpu)."""
    loc = [0]
    for n, _, _ in spec:
        loc.append(loc[-1] + n)
    return (torch.tensor(loc, dtype=torch.int32),
            torch.tensor([s[1] for s in spec], dtype=torch.int32),
            torch.tensor([s[2] for s in spec], dtype=torch.int32))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [96, 250, 1024, 2052, 5120, 9000])
def test_layer_norms(dtype, width):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(7, width, generator=g) * 3 + 1
    w = torch.rand(width, generator=g) + 0.5
    out = ops.layer_norm_stream(x.to(DEV), w.to(DEV), 1e-5, dtype)
    _close(out, ref.layer_norm_stream(x, w, 1e-5, dtype), dtype, "layer_norm_stream")

    a = (torch.randn(7, width, generator=g)).to(dtype)
    b = (torch.randn(7, width, generator=g)).to(dtype)
    ls = torch.rand(width, generator=g)
    nw = torch.rand(width, generator=g) + 0.5
    for bb in (None, b):
        xr = x.clone()
        ref.stream_add_layer_norm(xr, a, bb, 0.7, 0.4, w, ls, 1e-5)
        hr = ref.layer_norm_stream(xr, nw, 1e-5, dtype)
        xg = x.clone().to(DEV)
        hg = ops.stream_add_layer_norm(xg, a.to(DEV), None if bb is None else bb.to(DEV),
                                       0.7, 0.4, w.to(DEV), ls.to(DEV), 1e-5,
                                       (nw.to(DEV), 1e-5, dtype))
        _close(xg, xr, torch.float32 if dtype == torch.float32 else dtype, "stream")
        _close(hg, hr, dtype, "fused next norm")
    xg = x.clone().to(DEV)
    xr = x.clone()
    v = torch.randn(width, generator=g)
    ops.stream_add_vec(xg, a.float().to(DEV), v.to(DEV))
    ref.stream_add_vec(xr, a.float(), v)
    _close(xg, xr, torch.float32, "stream_add_vec")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gate_first", [True, False])
def test_gated_group_norm(dtype, gate_first):
    g = torch.Generator().manual_seed(2)
    y = torch.randn(5, 120, generator=g)
    wide = torch.randn(5, 300, generator=g).to(dtype)
    gate = wide[:, 100:220]
    w = torch.rand(120, generator=g) + 0.5
    for groups in (1, 3, 5):
        out = ops.gated_group_norm(y.to(DEV), wide.to(DEV)[:, 100:220], w.to(DEV), groups,
                                   1e-5, gate_first, dtype)
        _close(out, ref.gated_group_norm(y, gate, w, groups, 1e-5, gate_first, dtype),
               dtype, f"groups {groups}")
    # 16-byte paths: aligned gate slice, parts of 64 to 4096 values, and 6144
    y = torch.randn(3, 6144, generator=g)
    wide = torch.randn(3, 6144 + 128, generator=g).to(dtype)
    w = torch.rand(6144, generator=g) + 0.5
    for groups in (96, 12, 3, 2, 1):
        out = ops.gated_group_norm(y.to(DEV), wide.to(DEV)[:, 64:64 + 6144], w.to(DEV), groups,
                                   1e-5, gate_first, dtype)
        _close(out, ref.gated_group_norm(y, wide[:, 64:64 + 6144], w, groups, 1e-5, gate_first,
                                         dtype), dtype, f"wide groups {groups}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dims", [(5, 5, 24, 40), (6, 2, 32, 32), (4, 1, 72, 16), (3, 3, 10, 6),
                                  (8, 2, 128, 128), (2, 1, 256, 64), (2, 1, 32, 320), (1, 1, 8, 1000)])
def test_qk_norm_and_attention(dtype, dims):
    heads, kvh, dim, vdim = dims
    g = torch.Generator().manual_seed(3)
    bs, nblocks = 16, 40
    lens = [37, 300, 1]
    news = [5, 300, 1]
    t = sum(news)
    rows = heads * dim + kvh * (dim + vdim)
    proj = torch.randn(t, rows + 8, generator=g).to(dtype)
    qw = torch.rand(dim, generator=g) + 0.5
    kw = torch.rand(dim, generator=g) + 0.5
    kc = torch.randn(nblocks, bs, kvh, dim, generator=g).to(dtype)
    vc = torch.randn(nblocks, bs, kvh, vdim, generator=g).to(dtype)
    perm = torch.randperm(nblocks, generator=g).tolist()
    tables, slot_map, pos = [], [], []
    maxb = max((n + bs - 1) // bs for n in lens)
    for n, new in zip(lens, news):
        nb = (n + bs - 1) // bs
        blocks = [perm.pop() for _ in range(nb)]
        tables.append(blocks + [0] * (maxb - nb))
        for p in range(n - new, n):
            slot_map.append(blocks[p // bs] * bs + p % bs)
            pos.append(p)
    slot_map = torch.tensor(slot_map)
    pos = torch.tensor(pos)
    tables = torch.tensor(tables, dtype=torch.int32)

    def views(p):
        a = heads * dim
        b = a + kvh * dim
        return (p[:, :a].view(t, heads, dim), p[:, a:b].view(t, kvh, dim),
                p[:, b:rows].view(t, kvh, vdim))

    kc_r, vc_r = kc.clone(), vc.clone()
    q_r = ref.qk_norm_cache_write(*views(proj), qw, kw, 1e-5, pos, 0.5, 7, kc_r, vc_r, slot_map)
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    q_g = ops.qk_norm_cache_write(*views(proj.to(DEV)), qw.to(DEV), kw.to(DEV), 1e-5,
                                  pos.to(DEV), 0.5, 7, kc_g, vc_g, slot_map.to(DEV))
    _close(q_g, q_r, dtype, "q")
    _close(kc_g, kc_r, dtype, "k cache")
    _close(vc_g, vc_r, dtype, "v cache")

    # prompt portions: first two sequences; single query: the third
    npt = news[0] + news[1]
    qsl = torch.tensor([0, news[0], npt], dtype=torch.int32)
    sl = torch.tensor(lens[:2], dtype=torch.int32)
    want = ref.paged_attention(q_r[:npt], kc_r, vc_r, tables[:2], qsl, sl, 0.11)
    out = torch.empty((t, heads, vdim), dtype=dtype, device=DEV)
    ops._S.paged_attention_any(out[:npt], q_r[:npt].to(DEV), kc_g, vc_g, tables[:2].to(DEV),
                               qsl.to(DEV), sl.to(DEV), 0.11, max(news), 0, False, 0.0)
    _close(out[:npt], want, dtype, "prefill")
    sl1 = torch.tensor([lens[2], 0], dtype=torch.int32)      # second row: padding
    q1 = torch.cat([q_r[npt:], q_r[npt:]]).to(DEV)
    out1 = torch.full((2, heads, vdim), 7.0, dtype=dtype, device=DEV)
    bt1 = torch.cat([tables[2:], tables[2:]]).to(DEV)
    ops._S.paged_attention_any(out1, q1, kc_g, vc_g, bt1, None, sl1.to(DEV), 0.11, 1, 0, False, 0.0)
    want1 = ref.paged_attention(q_r[npt:], kc_r, vc_r, tables[2:], torch.tensor([0, 1], dtype=torch.int32),
                                sl1[:1], 0.11)
    _close(out1[:1], want1, dtype, "decode")
    assert float(out1[1].float().abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matrix_core_attention_dispatch(dtype):
    """Shapes the MFMA kernels take give the same attention as the any-shape
    kernel (through the public dispatch)."""
    if not ops.has_native():
        pytest.skip("_C not built")
    g = torch.Generator().manual_seed(4)
    heads, kvh, dim = 8, 2, 64
    bs, nblocks, n = 16, 24, 200
    q = torch.randn(n, heads, dim, generator=g).to(dtype).to(DEV)
    kc = torch.randn(nblocks, bs, kvh, dim, generator=g).to(dtype).to(DEV)
    vc = torch.randn(nblocks, bs, kvh, dim, generator=g).to(dtype).to(DEV)
    tables = torch.randperm(nblocks, generator=g)[: (n + bs - 1) // bs].to(torch.int32).view(1, -1).to(DEV)
    qsl = torch.tensor([0, n], dtype=torch.int32, device=DEV)
    sl = torch.tensor([n], dtype=torch.int32, device=DEV)
    a = torch.empty((n, heads, dim), dtype=dtype, device=DEV)
    b = torch.empty_like(a)
    ops.gqa_attention_prefill(q, kc, vc, tables, qsl, sl, 0.1, n, out=a)
    ops._S.paged_attention_any(b, q, kc, vc, tables, qsl, sl, 0.1, n, 0, False, 0.0)
    _close(a, b, dtype, "prefill dispatch")
    ops.gqa_attention_decode(q[-1:], kc, vc, tables, sl, 0.1, out=a[:1])
    _close(a[:1], b[-1:], dtype, "decode dispatch")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 4, 5])
def test_conv_bias_act_slice(dtype, taps):
    g = torch.Generator().manual_seed(5)
    width = 36
    spec = [(6, 6, 2), (1, 9, 0), (3, 4, -1), (2, 2, 1)]
    loc, lens, slots = _seqs(spec)
    t = int(loc[-1])
    wide = torch.randn(t, width + 20, generator=g).to(dtype)
    w = torch.randn(width, taps, generator=g)
    bias = torch.randn(width, generator=g)
    st = torch.randn(3, taps - 1, width, generator=g).to(dtype)
    for act in (None, "silu"):
        st_r, st_g = st.clone(), st.clone().to(DEV)
        want = ref.causal_conv_state(wide[:, 12:12 + width], w, st_r, loc, lens, slots, False, bias, act)
        got = ops.causal_conv_state(wide.to(DEV)[:, 12:12 + width], w.to(DEV), st_g, loc.to(DEV),
                                    lens.to(DEV), slots.to(DEV), False, bias.to(DEV), act)
        keep = torch.ones(t, dtype=torch.bool)
        keep[int(loc[2]):int(loc[3])] = False
        _close(got[keep.to(DEV)], want[keep], dtype, f"conv act={act}")
        assert float(got[~keep.to(DEV)].float().abs().max()) == 0.0
        _close(st_g[[0, 1, 2]], st_r[[0, 1, 2]], dtype, "conv state")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(4, 24, 16, 2), (3, 20, 40, 1), (2, 64, 128, 1), (5, 8, 6, 5), (2, 160, 128, 2),
                                   (1, 264, 24, 1)])
def test_ssd_scan(dtype, sizes):
    heads, vdim, nstate, groups = sizes
    g = torch.Generator().manual_seed(6)
    inner = heads * vdim
    spec = [(9, 9, 1), (1, 30, 0), (4, 12, 2), (1, 0, -1)]
    loc, lens, slots = _seqs(spec)
    t = int(loc[-1])
    xbc = (torch.randn(t, inner + 2 * groups * nstate, generator=g) * 0.5).to(dtype)
    wide = torch.randn(t, heads + 3, generator=g).to(dtype)
    dtb = torch.randn(heads, generator=g) - 2
    alog = torch.rand(heads, generator=g) * 2
    dsk = torch.randn(heads, generator=g)
    st = torch.randn(3, heads, vdim, nstate, generator=g)
    st_r, st_g = st.clone(), st.clone().to(DEV)
    want = ref.ssd_scan(xbc, wide[:, 2:2 + heads], dtb, alog, dsk, st_r, loc, lens, slots,
                        heads, vdim, nstate, groups)
    got = ops.ssd_scan(xbc.to(DEV), wide.to(DEV)[:, 2:2 + heads], dtb.to(DEV), alog.to(DEV),
                       dsk.to(DEV), st_g, loc.to(DEV), lens.to(DEV), slots.to(DEV),
                       heads, vdim, nstate, groups)
    _close(got, want, torch.float32, "ssd y")
    _close(st_g, st_r, torch.float32, "ssd state")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(3, 16, 24), (2, 40, 20), (1, 128, 64), (4, 8, 136), (1, 256, 72), (2, 64, 256)])
def test_mlstm_scan(dtype, sizes):
    heads, dim, vdim = sizes
    g = torch.Generator().manual_seed(7)
    spec = [(11, 11, 0), (1, 40, 2), (3, 8, 1), (1, 0, -1)]
    loc, lens, slots = _seqs(spec)
    t = int(loc[-1])
    rows = 2 * heads * dim + heads * vdim + 2 * heads
    proj = torch.randn(t, rows, generator=g).to(dtype)
    a, b = heads * dim, 2 * heads * dim
    c = b + heads * vdim

    def views(p):
        return (p[:, :a].view(t, heads, dim), p[:, a:b].view(t, heads, dim),
                p[:, b:c].view(t, heads, vdim), p[:, c:c + heads] * 4, p[:, c + heads:] * 4)

    ib = torch.randn(heads, generator=g)
    fb = torch.randn(heads, generator=g) + 2
    S = torch.randn(3, heads, vdim, dim, generator=g)
    N = torch.randn(3, heads, dim, generator=g)
    M = torch.randn(3, heads, generator=g)
    Sr, Nr, Mr = S.clone(), N.clone(), M.clone()
    Sg, Ng, Mg = S.clone().to(DEV), N.clone().to(DEV), M.clone().to(DEV)
    q, k, v, ip, fp = views(proj)
    want = ref.mlstm_scan(q, k, v, ip.contiguous(), fp.contiguous(), ib, fb, 6.0, dim ** -0.5,
                          Sr, Nr, Mr, loc, lens, slots)
    q, k, v, ip, fp = views(proj.to(DEV))
    got = ops.mlstm_scan(q, k, v, ip.contiguous(), fp.contiguous(), ib.to(DEV), fb.to(DEV), 6.0,
                         dim ** -0.5, Sg, Ng, Mg, loc.to(DEV), lens.to(DEV), slots.to(DEV))
    _close(got, want, torch.float32, "mlstm o")
    _close(Sg, Sr, torch.float32, "mlstm S")
    _close(Ng, Nr, torch.float32, "mlstm n")
    _close(Mg, Mr, torch.float32, "mlstm m")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [48, 300])
def test_rglru_scan(dtype, width):
    g = torch.Generator().manual_seed(8)
    spec = [(7, 7, 1), (1, 20, 0), (5, 9, 2), (1, 0, -1)]
    loc, lens, slots = _seqs(spec)
    t = int(loc[-1])
    u, rp, ip, yb = [torch.randn(t, width, generator=g).to(dtype) for _ in range(4)]
    rb, ibias = torch.randn(width, generator=g), torch.randn(width, generator=g)
    lam = torch.randn(width, generator=g)
    st = torch.randn(3, width, generator=g)
    st_r, st_g = st.clone(), st.clone().to(DEV)
    want = ref.rglru_scan(u, rp, ip, rb, ibias, lam, 8.0, yb, st_r, loc, lens, slots)
    got = ops.rglru_scan(u.to(DEV), rp.to(DEV), ip.to(DEV), rb.to(DEV), ibias.to(DEV),
                         lam.to(DEV), 8.0, yb.to(DEV), st_g, loc.to(DEV), lens.to(DEV),
                         slots.to(DEV))
    _close(got, want, dtype, "rglru out")
    _close(st_g, st_r, torch.float32, "rglru state")
