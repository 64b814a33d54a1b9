"""Fused decode + matrix-vector product against an fp64 product of the
reconstructed weights (floating point: tolerance stated per assertion)."""
import ctypes

import numpy as np
import pytest

from conftest import bf16_bits_normal, closed_form_recon, stress_bits

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _bf16_to_f64(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def _weight(rows, cols, kind, seed):
    bits = bf16_bits_normal(rows * cols, seed) if kind == "normal" else stress_bits(rows, cols, seed)
    if kind == "stress":  # keep the product finite: no Inf/NaN patterns
        bits = np.where(((bits >> 7) & 0xFF) == 0xFF, np.uint16(0x3C00), bits)
    return bits


def _gemv(mgr, handles, x, biases):
    be = mgr._be
    names = (ctypes.c_char_p * len(handles))(*[h.encode() for h in handles])
    outs = [torch.full((int(np.prod(mgr.meta_dict[h])) // x.numel(),), 7.0, dtype=torch.bfloat16, device="cuda")
            for h in handles]
    be.gemv_batch(names, x, biases, outs)
    torch.cuda.synchronize()
    return outs


def _check(y, w_bits, x, bias, s):
    rows = y.numel()
    w = _bf16_to_f64(closed_form_recon(w_bits, s)).reshape(rows, -1)
    xv = x.double().cpu().numpy()
    ref = w @ xv
    if bias is not None:
        ref = ref + bias.double().cpu().numpy()
    got = y.double().cpu().numpy()
    # bf16 output: half an ulp is 2^-9 relative; fp32 partial sums add a little
    # relative to the sum of magnitudes
    tol = 2.0 ** -8 * np.abs(ref) + 1e-5 * (np.abs(w) @ np.abs(xv)) + 2.0 ** -36
    assert np.all(np.abs(got - ref) <= tol), float(np.max(np.abs(got - ref) / tol))


@pytest.mark.parametrize("s", [7, 3, 0])
@pytest.mark.parametrize("rows,cols,kind,lane", [
    (64, 512, "normal", 0), (1000, 1024, "stress", 0), (4096, 4096, "normal", 0),
    (333, 14336, "normal", 0), (512, 2048, "normal", 128), (96, 3584, "stress", "auto"),
])
def test_gemv_matches_fp64_product(rows, cols, kind, lane, s):
    import neuzip_amd

    mgr = neuzip_amd.Manager(precision=s, lane_symbols=lane)
    bits = _weight(rows, cols, kind, seed=rows + s)
    w = torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16).view(rows, cols)
    h = mgr.write(w)
    g = torch.Generator(device="cuda").manual_seed(rows)
    x = torch.randn(cols, device="cuda", generator=g).to(torch.bfloat16)
    bias = torch.randn(rows, device="cuda", generator=g).to(torch.bfloat16)
    print(f"case gemv {rows}x{cols} {kind} lane={lane} s={s}", flush=True)
    (y,) = _gemv(mgr, [h], x, None)
    _check(y, bits, x, None, s)
    (yb,) = _gemv(mgr, [h], x, [bias])
    _check(yb, bits, x, bias, s)
    # deterministic, and the accumulators are clean again after every call
    (y2,) = _gemv(mgr, [h], x, None)
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))
    mgr._be.check()


@pytest.mark.parametrize("rows,cols", [(14336, 4096), (4096, 4096), (2048, 14336)])
def test_gemv_at_the_geometries_chosen_per_tensor(rows, cols):
    """Per-tensor geometry: segments of 14 336 elements (rows straddle them), of
    4096 (one row each, stored directly) and of 7168 (a row spans two or three)."""
    import neuzip_amd

    mgr = neuzip_amd.Manager(precision=7, lane_symbols="auto")
    bits = _weight(rows, cols, "normal", seed=rows)
    w = torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16).view(rows, cols)
    h = mgr.write(w)
    g = torch.Generator(device="cuda").manual_seed(cols)
    x = torch.randn(cols, device="cuda", generator=g).to(torch.bfloat16)
    print(f"case gemv auto {rows}x{cols}", flush=True)
    (y,) = _gemv(mgr, [h], x, None)
    _check(y, bits, x, None, 7)
    (y2,) = _gemv(mgr, [h], x, None)
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))
    assert torch.equal(mgr.read(h), w)
    mgr._be.check()


def test_gemv_batch_equals_single_calls_and_rejects_bad_shapes():
    import neuzip_amd

    mgr = neuzip_amd.Manager()
    cols = 1024
    shapes = [(256, cols), (64, cols), (1024, cols), (8, cols)]
    ws, hs = [], []
    for i, (r, c) in enumerate(shapes):
        bits = bf16_bits_normal(r * c, seed=40 + i)
        w = torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16).view(r, c)
        ws.append(w)
        hs.append(mgr.write(w))
    x = torch.randn(cols, device="cuda").to(torch.bfloat16)
    biases = [None, torch.randn(64, device="cuda").to(torch.bfloat16), None, None]
    together = _gemv(mgr, hs, x, biases)
    for h, b, y in zip(hs, biases, together):
        (alone,) = _gemv(mgr, [h], x, [b])
        assert torch.equal(alone.view(torch.int16), y.view(torch.int16))
    # in_features must divide the tensor and be a multiple of 512; nothing is written otherwise
    be = mgr._be
    odd = mgr.write(torch.zeros(3, 700, dtype=torch.bfloat16, device="cuda"))
    for handle, xin in ((odd, torch.zeros(700, dtype=torch.bfloat16, device="cuda")),
                        (hs[0], torch.zeros(1536, dtype=torch.bfloat16, device="cuda"))):
        out = torch.full((4096,), 7.0, dtype=torch.bfloat16, device="cuda")
        names = (ctypes.c_char_p * 1)(handle.encode())
        with pytest.raises(ValueError):
            be.gemv_batch(names, xin, None, [out])
        torch.cuda.synchronize()
        assert bool((out == 7.0).all())
    be.check()


def test_gemv_non_finite_input_gives_non_finite_rows_then_recovers():
    import neuzip_amd

    mgr = neuzip_amd.Manager()
    for rows, cols in ((128, 512), (64, 14336)):  # rows inside one segment / rows shared by segments
        bits = bf16_bits_normal(rows * cols, seed=3)
        w = torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16).view(rows, cols)
        h = mgr.write(w)
        x = torch.randn(cols, device="cuda").to(torch.bfloat16)
        bad = x.clone()
        bad[17] = float("inf")
        (y,) = _gemv(mgr, [h], bad, None)
        # a row inside one segment carries the infinity like a plain product; a row summed
        # across segments is flagged and comes out as NaN
        assert not bool(torch.isfinite(y.float()).any())
        (y,) = _gemv(mgr, [h], x, None)  # flags, counts and sums were cleared
        _check(y, bits, x, None, 7)
    mgr._be.check()


class _Attn(torch.nn.Module):
    def __init__(self, d):
        super().__init__()
        self.q = torch.nn.Linear(d, d, bias=False)
        self.k = torch.nn.Linear(d, d // 2, bias=True)
        self.v = torch.nn.Linear(d, d // 2, bias=False)
        self.o = torch.nn.Linear(d, d, bias=True)

    def forward(self, x):
        q, k, v = self.q(x), self.k(x), self.v(x)
        return x + self.o(q * torch.cat((k, v), dim=-1))


def test_fused_gemv_module_groups_and_graph_replay():
    import neuzip_amd

    torch.manual_seed(11)
    model = torch.nn.Sequential(_Attn(512), _Attn(512)).to(torch.bfloat16)
    for p in model.parameters():
        p.data.normal_(0, 0.05)
    mgr = neuzip_amd.Manager()
    mgr.convert(model)
    model = model.cuda()
    xs = [torch.randn(1, 1, 512, device="cuda").to(torch.bfloat16) for _ in range(4)]
    x_static = torch.zeros_like(xs[0])
    with torch.no_grad():
        wants = [model(x) for x in xs]
        many = torch.randn(3, 512, device="cuda").to(torch.bfloat16)
        want_many = model(many)
        fused = neuzip_amd.FusedGemv(mgr, model)
        fused.trace(lambda: model(xs[0]))
        assert sorted(len(g.handles) for g in fused._groups) == [1, 1, 3, 3]
        with fused:
            eager = [model(x) for x in xs]
            for got, want in zip(eager, wants):
                # every Linear output is rounded to bf16 on both paths: a few ulps through two blocks
                assert torch.allclose(got.float(), want.float(), rtol=3e-2, atol=3e-2)
            assert torch.equal(model(many), want_many)  # several rows: the ordinary path
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                model(x_static)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                y_static = model(x_static)
            for x, want in zip(xs, eager):
                x_static.copy_(x)
                g.replay()
                got = y_static.clone()
                torch.cuda.synchronize()
                assert torch.equal(got, want)  # the fused path itself is deterministic
                (x * 2).sum().item()
        assert torch.equal(model(xs[0]), wants[0])  # hook removed again
    mgr._be.check()


def test_raw_chunks_through_product_gather_and_normalizers():
    """Incompressible exponents (all 255 finite exponent bytes equally likely) are
    stored raw; the fused product, the row gather and the normalized decode take
    their own path through such chunks."""
    import neuzip_amd

    rng = np.random.default_rng(17)
    rows, cols = 384, 1024
    bits = ((rng.integers(0, 255, rows * cols).astype(np.uint16) << 7) |
            rng.integers(0, 128, rows * cols).astype(np.uint16) |
            (rng.integers(0, 2, rows * cols).astype(np.uint16) << 15))
    w = torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16).view(rows, cols)
    for norm in (0, 64):
        mgr = neuzip_amd.Manager(normalizer_size=norm)
        h = mgr.write(w)
        assert mgr._be.exp_bytes(h) > rows * cols  # raw: no smaller than the exponent bytes
        full = mgr.read(h)
        if norm == 0:
            assert torch.equal(full.view(torch.int16), w.view(torch.int16))
        idx = torch.tensor([0, rows - 1, 17, 200], device="cuda")
        assert torch.equal(mgr.gather_rows(h, idx).view(torch.int16), full[idx].view(torch.int16))
        # one non-zero activation small enough to keep every product finite and in range
        x = torch.zeros(cols, dtype=torch.bfloat16, device="cuda")
        x[321] = 2.0 ** -120
        (y,) = _gemv(mgr, [h], x, None)
        ref = full[:, 321].double() * 2.0 ** -120
        # the sums are resolved to 2^-40; the bf16 result to half a unit in the last place
        assert bool(((y.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 2.0 ** -40).all())
        mgr._be.check()


def test_group_geometry_is_refitted_and_results_stay_the_same():
    """FusedGemv.trace stores the matrices of a group again with one geometry
    chosen for the group (manager with per-tensor geometry); later writes under
    those handles keep it; the stored values do not change."""
    import neuzip_amd

    class Pair(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = torch.nn.Linear(2048, 6144, bias=False)
            self.b = torch.nn.Linear(2048, 6144, bias=True)

        def forward(self, x):
            return self.a(x) + self.b(x)

    torch.manual_seed(11)
    model = Pair().to(torch.bfloat16)
    for p in model.parameters():
        p.data.normal_(0, 0.02)
    mgr = neuzip_amd.Manager(lane_symbols="auto")
    mgr.convert(model)
    model = model.cuda()
    ha, hb = model.a.weight._handle, model.b.weight._handle
    wa, wb = mgr.read(ha).clone(), mgr.read(hb).clone()
    before = mgr._be.geometry(ha)
    x = torch.randn(1, 2048, device="cuda", dtype=torch.bfloat16)
    fused = neuzip_amd.FusedGemv(mgr, model)
    with torch.no_grad():
        want = model(x)
        fused.trace(lambda: model(x))
        after = mgr._be.geometry(ha)
        print(f"geometry {before} -> {after}", flush=True)
        assert after == mgr._be.geometry(hb) and after[0] == 512 * after[1]
        assert torch.equal(mgr.read(ha), wa) and torch.equal(mgr.read(hb), wb)
        with fused:
            got = model(x)
        assert torch.allclose(got.float(), want.float(), rtol=2e-2, atol=2e-2)
        mgr.write(wa * 2, ha)                      # a later write keeps the group's geometry
        assert mgr._be.geometry(ha) == after and torch.equal(mgr.read(ha), wa * 2)
    mgr._be.check()


@pytest.mark.parametrize("s", [7, 3])
@pytest.mark.parametrize("m_rows", [2, 3, 4, 5, 8])
def test_several_activation_rows_equal_the_one_row_calls(m_rows, s):
    """nz_manager_gemv_rows_batch: every weight is decoded once and multiplied with
    up to eight activation rows.  Each output row is, bit for bit, what the one-row
    call gives for that activation row (same order of additions per row), so it is
    within the same tolerance of the fp64 product; matrices whose rows lie inside
    a segment, straddle segments, and a group of matrices in one launch."""
    import neuzip_amd

    mgr = neuzip_amd.Manager(precision=s)
    be = mgr._be
    cols = 4096
    shapes = [(4096, cols), (96, cols), (1030, cols)]
    bits = [_weight(r, c, "normal" if i != 1 else "stress", seed=70 + i + s) for i, (r, c) in enumerate(shapes)]
    hs = [mgr.write(torch.from_numpy(b.view(np.int16).copy()).cuda().view(torch.bfloat16).view(r, c))
          for b, (r, c) in zip(bits, shapes)]
    g = torch.Generator(device="cuda").manual_seed(m_rows)
    x = torch.randn(m_rows, cols, device="cuda", generator=g).to(torch.bfloat16)
    biases = [None, torch.randn(96, device="cuda", generator=g).to(torch.bfloat16), None]
    names = (ctypes.c_char_p * len(hs))(*[h.encode() for h in hs])
    print(f"case rows={m_rows} s={s}", flush=True)
    outs = [torch.full((m_rows, r), 7.0, dtype=torch.bfloat16, device="cuda") for r, _ in shapes]
    be.gemv_batch(names, x, biases, outs, m_rows)
    torch.cuda.synchronize()
    for i, (h, b) in enumerate(zip(hs, biases)):
        for m in range(m_rows):
            (one,) = _gemv(mgr, [h], x[m].contiguous(), [b])
            assert torch.equal(one.view(torch.int16), outs[i][m].view(torch.int16)), (i, m)
            _check(outs[i][m], bits[i], x[m], b, s)
    # again, with the matrices one by one: the accumulators were left clean
    for i, h in enumerate(hs):
        out = torch.full((m_rows, shapes[i][0]), 7.0, dtype=torch.bfloat16, device="cuda")
        be.gemv_batch((ctypes.c_char_p * 1)(h.encode()), x, [biases[i]], [out], m_rows)
        assert torch.equal(out.view(torch.int16), outs[i].view(torch.int16))
    # more than eight rows, or rows with a manager that has normalizers: refused, nothing written
    xbig = torch.zeros(9, cols, dtype=torch.bfloat16, device="cuda")
    sink = torch.full((9, 4096), 7.0, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="activation rows"):
        be.gemv_batch((ctypes.c_char_p * 1)(hs[0].encode()), xbig, None, [sink], 9)
    assert bool((sink == 7.0).all())
    be.check()


def test_linear_with_a_few_rows_takes_the_fused_product(oracle):
    """Manager.linear with a 2-D (or batched) input of two to eight rows: served by
    the fused product (equal to the one-row calls), nine rows and more by
    decompress-then-GEMM (equal to torch's linear on the decoded weight); Linears
    that share their input are still recognised and launched together."""
    import neuzip_amd

    mgr = neuzip_amd.Manager(precision=7)
    cols = 2048
    ws = [(torch.randn(r, cols, device="cuda") * 0.02).to(torch.bfloat16) for r in (1536, 512, 512)]
    bias = torch.randn(1536, device="cuda").to(torch.bfloat16)
    hs = [mgr.write(w) for w in ws]
    with torch.no_grad():
        for shape in ((4, cols), (2, 3, cols), (1, 8, cols)):
            x = torch.randn(*shape, device="cuda").to(torch.bfloat16)
            for rep in range(3):  # the second pass has learned that the three share their input
                got = [mgr.linear(hs[0], x, bias), mgr.linear(hs[1], x), mgr.linear(hs[2], x)]
                flat = x.reshape(-1, cols)
                for k, (h, w, b) in enumerate(zip(hs, ws, (bias, None, None))):
                    assert got[k].shape == x.shape[:-1] + (w.shape[0],)
                    for m in range(flat.shape[0]):
                        mgr.group_rows = False
                        one = mgr.linear(h, flat[m].contiguous(), b)
                        mgr.group_rows = True
                        assert torch.equal(one, got[k].reshape(-1, w.shape[0])[m]), (shape, rep, k, m)
        assert sorted(len(r[0]) for r in mgr._be._runs.values()) == [3]
        x9 = torch.randn(9, cols, device="cuda").to(torch.bfloat16)
        assert torch.equal(mgr.linear(hs[0], x9, bias), torch.nn.functional.linear(x9, ws[0], bias))
    mgr._be.check()


def test_runs_of_calls_that_share_their_activation_are_learned_and_checked():
    """Manager.linear recognises Linears called back to back with the same
    activation tensor and serves them with one launch from the second time on.
    A result computed ahead is handed out only for the very same tensor object,
    unmodified, and the same bias; anything else falls back to a launch of its
    own and the run is forgotten.  Every result equals the single launch's."""
    import neuzip_amd

    cols = 1024
    ws = [(torch.randn(r, cols, device="cuda") * 0.02).to(torch.bfloat16) for r in (768, 256, 256, 512)]
    bias = torch.randn(256, device="cuda").to(torch.bfloat16)

    def fresh():
        mgr = neuzip_amd.Manager(precision=7)
        return mgr, [mgr.write(w) for w in ws]

    def alone(mgr, h, x, b=None):
        was = mgr.group_rows
        mgr.group_rows = False
        try:
            return mgr.linear(h, x, b)
        finally:
            mgr.group_rows = was

    with torch.no_grad():
        # learned on the first pass, grouped from the second: same numbers, one run of three
        mgr, hs = fresh()
        for rep in range(3):
            x = torch.randn(cols, device="cuda").to(torch.bfloat16)
            y = [mgr.linear(hs[0], x), mgr.linear(hs[1], x, bias), mgr.linear(hs[2], x)]
            mgr.linear(hs[3], torch.randn(cols, device="cuda").to(torch.bfloat16))  # another input: not part of the run
            for k, b in ((0, None), (1, bias), (2, None)):
                assert torch.equal(y[k], alone(mgr, hs[k], x, b)), (rep, k)
        assert [r[0] for r in mgr._be._runs.values()] == [hs[:3]]
        assert not mgr._be._parked

        # the activation is modified in place between two calls of a learned run
        x = torch.randn(cols, device="cuda").to(torch.bfloat16)
        y0 = mgr.linear(hs[0], x)          # computes all three ahead
        x.mul_(2)
        y1 = mgr.linear(hs[1], x, bias)    # must see the new values
        assert torch.equal(y1, alone(mgr, hs[1], x, bias))
        assert hs[0] not in mgr._be._runs and not mgr._be._parked  # forgotten for good
        for rep in range(2):                # ... and not learned again
            x = torch.randn(cols, device="cuda").to(torch.bfloat16)
            mgr.linear(hs[0], x), mgr.linear(hs[1], x, bias), mgr.linear(hs[2], x)
        assert not mgr._be._runs

        # an equal but different tensor object, and another bias, are not taken for the learned ones
        mgr, hs = fresh()
        for rep in range(2):
            x = torch.randn(cols, device="cuda").to(torch.bfloat16)
            mgr.linear(hs[0], x), mgr.linear(hs[1], x, bias), mgr.linear(hs[2], x)
        x = torch.randn(cols, device="cuda").to(torch.bfloat16)
        mgr.linear(hs[0], x)
        other = torch.randn(cols, device="cuda").to(torch.bfloat16)
        assert torch.equal(mgr.linear(hs[1], other, bias), alone(mgr, hs[1], other, bias))
        mgr, hs = fresh()
        for rep in range(2):
            x = torch.randn(cols, device="cuda").to(torch.bfloat16)
            mgr.linear(hs[0], x), mgr.linear(hs[1], x, bias), mgr.linear(hs[2], x)
        x = torch.randn(cols, device="cuda").to(torch.bfloat16)
        mgr.linear(hs[0], x)
        bias2 = bias.clone().add_(1)
        assert torch.equal(mgr.linear(hs[1], x, bias2), alone(mgr, hs[1], x, bias2))

        # a weight of the run is rewritten between two calls: nothing computed ahead survives the write
        mgr, hs = fresh()
        for rep in range(2):
            x = torch.randn(cols, device="cuda").to(torch.bfloat16)
            mgr.linear(hs[0], x), mgr.linear(hs[1], x, bias), mgr.linear(hs[2], x)
        x = torch.randn(cols, device="cuda").to(torch.bfloat16)
        mgr.linear(hs[0], x)
        w_new = (ws[1].float() * 1.5).to(torch.bfloat16)
        mgr.write(w_new, hs[1])
        got = mgr.linear(hs[1], x, bias)
        assert torch.equal(got, alone(mgr, hs[1], x, bias))
        assert not torch.equal(got, torch.zeros_like(got))
        # ... and the learned run goes on with the new weight
        x = torch.randn(cols, device="cuda").to(torch.bfloat16)
        y = [mgr.linear(hs[0], x), mgr.linear(hs[1], x, bias), mgr.linear(hs[2], x)]
        assert torch.equal(y[1], alone(mgr, hs[1], x, bias))

        # a member called out of order, without the first one: a launch of its own
        x = torch.randn(cols, device="cuda").to(torch.bfloat16)
        assert torch.equal(mgr.linear(hs[2], x), alone(mgr, hs[2], x))
        mgr._be.check()


def test_dense_weights_asked_for_in_a_repeating_order_share_decode_launches():
    """More rows than the fused product takes: decompress-then-GEMM.  The order in
    which dense weights are asked for is learned, and a request that finds nothing
    waiting decodes the handles expected next in the same launch.  Results equal
    torch's linear on the stored weights bit for bit, whatever was decoded ahead:
    a write drops the weight that waits for its handle, an unforeseen request
    drops all that wait, and a manager whose order does not repeat stops."""
    import neuzip_amd

    cols = 1024
    ws = [(torch.randn(r, cols, device="cuda") * 0.02).to(torch.bfloat16) for r in (768, 256, 256, 512)]
    bias = torch.randn(256, device="cuda").to(torch.bfloat16)
    mgr = neuzip_amd.Manager(precision=7)
    hs = [mgr.write(w) for w in ws]
    calls = []
    real = mgr._be.read_batch

    def counting(plan, outs):
        calls.append(plan[2])
        return real(plan, outs)

    def lin(x, k, b=None, w=None):
        got = mgr.linear(hs[k], x, b)
        assert torch.equal(got, torch.nn.functional.linear(x, ws[k] if w is None else w, b)), k
        return got

    mgr._be.read_batch = counting
    try:
        with torch.no_grad():
            for rep in range(3):
                x = torch.randn(3, 16, cols, device="cuda").to(torch.bfloat16)
                lin(x, 0), lin(x, 1, bias), lin(x, 2)
                lin(torch.randn(40, cols, device="cuda").to(torch.bfloat16), 3)
            # pass one learns; in pass two the second request knows what follows (the four tensors
            # are far too small to fill the device, so the launch takes all of them, the first
            # weight of the next pass included); pass three finds that one waiting
            assert calls == [4, 4]
            assert mgr._be.ahead_stats() == (5, 0)
            # the runs of calls that share their activation were learned on the way, for single rows
            assert [r[0] for r in mgr._be._runs.values()] == [hs[:3]]
            x1 = torch.randn(cols, device="cuda").to(torch.bfloat16)
            y1 = [mgr.linear(hs[0], x1), mgr.linear(hs[1], x1, bias), mgr.linear(hs[2], x1)]
            mgr.group_rows = False
            assert all(torch.equal(a, mgr.linear(h, x1, b)) for a, h, b in zip(y1, hs, (None, bias, None)))
            mgr.group_rows = True

            # a rewrite while the old weight waits: the next request sees the new one
            x = torch.randn(12, cols, device="cuda").to(torch.bfloat16)
            waiting = lambda: mgr._be._order.waiting()
            assert waiting() == {hs[0]}
            lin(x, 0), lin(x, 1, bias)
            assert waiting() == {hs[2], hs[3], hs[0]}
            w_new = (ws[2].float() * 0.5).to(torch.bfloat16)
            mgr.write(w_new, hs[2])
            assert waiting() == {hs[3], hs[0]}
            lin(x, 2, w=w_new)                      # decoded again, on its own: the others go on waiting
            ws[2] = w_new
            assert waiting() == {hs[3], hs[0]}
            lin(x, 3), lin(x, 0)
            assert not waiting()
            lin(x, 1, bias)                         # the walk that lost a weight to the write ends in front of
            assert not waiting()                    # that place the next time (and grows again from there)
            lin(x, 2)
            assert waiting() == {hs[3], hs[0], hs[1]}
            # a request that was not foreseen: served by a decode of its own, what waited is dropped
            w4 = (torch.randn(128, cols, device="cuda") * 0.02).to(torch.bfloat16)
            h4 = mgr.write(w4)
            wasted = mgr._be.ahead_stats()[1]
            assert torch.equal(mgr.linear(h4, x), torch.nn.functional.linear(x, w4))
            assert not waiting() and mgr._be.ahead_stats()[1] == wasted + 3
            # decoded on one stream, asked for on another
            lin(x, 3), lin(x, 0)
            assert waiting() == {hs[1], hs[2], h4, hs[3]}  # the new handle has taken its place in the learned order
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                y = mgr.linear(hs[1], x, bias)
            side.synchronize()
            assert torch.equal(y, torch.nn.functional.linear(x, ws[1], bias))
            torch.cuda.current_stream().wait_stream(side)
            # switched off: every request decodes its own tensor
            mgr.decode_ahead = False
            assert not mgr._be._order.waiting()
            n = len(calls)
            for rep in range(2):
                lin(x, 0), lin(x, 1, bias), lin(x, 2), lin(x, 3)
            assert len(calls) == n
            mgr._be.check()

            # an order that does not repeat: still the right numbers, and the manager stops decoding ahead
            mgr2 = neuzip_amd.Manager(precision=7)
            h2 = [mgr2.write(w) for w in ws]
            gen = torch.Generator().manual_seed(5)
            for rep in range(80):
                for k in torch.randperm(4, generator=gen).tolist():
                    got = mgr2.linear(h2[k], x)
                    assert torch.equal(got, torch.nn.functional.linear(x, ws[k])), (rep, k)
            assert mgr2._be._order.paused  # requests are served one by one for a while
            mgr2._be.check()
    finally:
        del mgr._be.read_batch
    mgr._be.check()


def test_backward_of_compressed_linears_takes_weights_decoded_ahead():
    """Training through converted Linears with nothing but the reference's calls:
    the backward pass asks for the weights in reverse and finds them decoded
    ahead from its second step on.  Outputs and gradients equal, bit for bit,
    those of a manager that decodes every weight on its own, and the dense
    model's to rounding."""
    import copy

    import neuzip_amd

    torch.manual_seed(3)
    dense = torch.nn.Sequential(*[torch.nn.Linear(512, 512, bias=(k % 2 == 0)) for k in range(6)]).cuda().bfloat16()
    mgr_a, mgr_b = neuzip_amd.Manager(precision=7), neuzip_amd.Manager(precision=7)
    mgr_b.decode_ahead = False
    comp_a, comp_b = mgr_a.convert(copy.deepcopy(dense)), mgr_b.convert(copy.deepcopy(dense))
    packed_a = [m._p for m in comp_a.modules() if isinstance(m, neuzip_amd.nn.Linear)]
    packed_b = [m._p for m in comp_b.modules() if isinstance(m, neuzip_amd.nn.Linear)]
    assert len(packed_a) == 6
    for step in range(4):
        x = torch.randn(24, 512, device="cuda").to(torch.bfloat16)
        xd, xa, xb = (x.clone().requires_grad_(True) for _ in range(3))
        yd, ya, yb = dense(xd), comp_a(xa), comp_b(xb)
        assert torch.equal(ya, yb), step
        for y in (yd, ya, yb):
            y.float().square().mean().backward()
        assert torch.equal(xa.grad, xb.grad), step
        torch.testing.assert_close(xa.grad.float(), xd.grad.float(), rtol=2e-2, atol=1e-6)
        for lin_d, pa, pb in zip(dense, packed_a, packed_b):
            assert torch.equal(pa._gradient, pb._gradient), step
            torch.testing.assert_close(pa._gradient.view_as(lin_d.weight.grad).float(), lin_d.weight.grad.float(),
                                       rtol=2e-2, atol=1e-6)
            lin_d.weight.grad = None
            pa._gradient = pb._gradient = None
        if step == 2:  # a weight changes between two steps: every model takes the new one
            with torch.no_grad():
                w = dense[3].weight.mul_(0.5)
                mgr_a.write(w, packed_a[3]._handle)
                mgr_b.write(w, packed_b[3]._handle)
    hits, waste = mgr_a._be.ahead_stats()
    assert hits >= 20 and waste == 0, (hits, waste)
    assert mgr_b._be.ahead_stats() == (0, 0)
    mgr_a._be.check()
    mgr_b._be.check()
