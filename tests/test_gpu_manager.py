"""GPU: the Manager / nn / ops surface on the native backend, against the
oracle's reconstruction and plain torch layers (neuzip/binding.py:55-111,
neuzip/nn/linear.py, neuzip/ops/linear.py, neuzip/__init__.py:25-35)."""
from functools import partial

import numpy as np
import pytest

from conftest import chunk_entropy_bytes, bf16_bits_normal, closed_form_recon, stress_bits

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def bits_of(t):
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1)


def from_bits(bits, shape, device="cuda"):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).reshape(shape).to(device)


@pytest.mark.parametrize("precision", (7, 3, 1, 0))
def test_write_read_size(oracle, precision):
    import neuzip_amd

    mgr = neuzip_amd.Manager(precision=precision)
    shapes = [(4096, 1024), (3, 5, 7), (1,), (513, 129), (0,)]
    handles = []
    for i, shp in enumerate(shapes):
        n = int(np.prod(shp))
        w = from_bits(bf16_bits_normal(n, seed=i + precision), shp)
        h = mgr.write(w)
        handles.append(h)
        assert h == str(i)  # auto handles are "0", "1", ... (binding.py:75-76)
        out = mgr.read(h)
        assert out.shape == torch.Size(shp) and out.dtype == torch.bfloat16 and not out.requires_grad
        assert np.array_equal(bits_of(out), oracle.reconstruct(bits_of(w), precision))
        assert mgr._be.geometry(h) == (_default_geometry(n) if n else (131072, 256))  # per tensor, inside the size budget
        o_comp, o_packed = oracle.compress_bf16(bits_of(w), precision, *mgr._be.geometry(h))
        assert mgr.size(h) == o_comp.size + o_packed.size  # exponents + packed bytes held
        assert mgr._be.packed_bytes(h) == o_packed.size
    assert mgr.size("nope") == 0  # cuda/high_level.cu:209-211
    with pytest.raises(KeyError):
        mgr.read("nope")
    with pytest.raises(RuntimeError, match="Data not found"):
        mgr._be.read("nope")
    mgr._be.check()


def test_overwrite_same_handle_and_named_handles(oracle):
    import neuzip_amd

    mgr = neuzip_amd.Manager()
    a = from_bits(bf16_bits_normal(70_000, 1), (70_000,))
    b = from_bits(bf16_bits_normal(10_000, 2), (100, 100))
    assert mgr.write(a, "w") == "w"
    assert mgr.write(b, "w") == "w"  # erase + insert (cuda/high_level.cu:137-142)
    assert torch.equal(mgr.read("w"), b)
    assert mgr.write(a) == "1"  # len(meta_dict) == 1
    assert torch.equal(mgr.read("1"), a)
    for _ in range(3):  # rewrite in place with fresh values, as the update hook does
        a = a * 1.01
        mgr.write(a, "1")
        assert torch.equal(mgr.read("1"), a)


def test_dtype_and_device_handling():
    import neuzip_amd

    mgr = neuzip_amd.Manager()
    with pytest.raises(RuntimeError, match="Unsupported data type"):
        mgr.write(torch.zeros(8, dtype=torch.float32, device="cuda"))
    with pytest.raises(RuntimeError, match="Unsupported data type"):
        mgr.write(torch.zeros(8, dtype=torch.float16, device="cuda"))
    cpu = torch.randn(33, 77).to(torch.bfloat16)
    h = mgr.write(cpu)  # host tensors are moved to the GPU (cuda/high_level.cu:133-135)
    out = mgr.read(h)
    assert out.is_cuda and torch.equal(out.cpu(), cpu)
    # non-contiguous and oddly offset views
    base = torch.randn(64, 64, device="cuda").to(torch.bfloat16)
    h2 = mgr.write(base.t())
    assert torch.equal(mgr.read(h2), base.t())
    flat = torch.randn(1001, device="cuda").to(torch.bfloat16)
    h3 = mgr.write(flat[1:])
    assert torch.equal(mgr.read(h3), flat[1:])


def test_split_api(oracle):
    import neuzip_amd

    mgr = neuzip_amd.Manager(precision=3)  # split always uses 7 kept bits (cuda/high_level.cu:289)
    w = from_bits(bf16_bits_normal(3 * 1000, 5), (3, 1000))
    e, f = mgr.split(w)
    assert e.shape == w.shape and f.shape == w.shape and e.dtype == torch.uint8 and f.dtype == torch.uint8
    oe, of = oracle.split(bits_of(w), 7)
    assert np.array_equal(e.cpu().numpy().reshape(-1), oe)
    assert np.array_equal(f.cpu().numpy().reshape(-1), of)


@pytest.mark.parametrize("precision", (7, 3))
@pytest.mark.parametrize("bias", (True, False))
def test_linear_forward_backward(oracle, precision, bias):
    import neuzip_amd

    torch.manual_seed(0)
    mgr = neuzip_amd.Manager(precision=precision)
    dense = torch.nn.Linear(256, 384, bias=bias).to(torch.bfloat16)
    dense.weight.data.normal_(0, 0.02)
    w_rec = from_bits(oracle.reconstruct(bits_of(dense.weight.data), precision), (384, 256))
    model = torch.nn.Sequential(dense)
    mgr.convert(model)
    model = model.cuda()
    lin = model[0]
    assert isinstance(lin, neuzip_amd.nn.Linear) and lin.weight.numel() == 0
    assert torch.equal(lin.weight(), w_rec)
    for shape in ((7, 256), (2, 5, 256)):
        x = torch.randn(*shape, device="cuda", dtype=torch.bfloat16)
        x1, x2 = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
        y1 = lin(x1)
        y2 = torch.nn.functional.linear(x2, w_rec, lin.bias)
        assert torch.equal(y1, y2)
        g = torch.randn_like(y1)
        lin.weight._gradient = None
        y1.backward(g)
        wr = w_rec.clone().requires_grad_(True)
        torch.nn.functional.linear(x2, wr, lin.bias).backward(g)
        assert torch.equal(x1.grad, x2.grad)
        assert torch.allclose(lin.weight._gradient.float(), wr.grad.float(), rtol=1e-2, atol=1e-2)
        assert lin.weight.grad.numel() == 0


def _toy(seed):
    torch.manual_seed(seed)
    m = torch.nn.Sequential(torch.nn.Linear(64, 128), torch.nn.GELU(), torch.nn.Linear(128, 64, bias=False)).to(torch.bfloat16)
    for p in m.parameters():
        p.data.normal_(0, 0.02)
    return m


class _Sched:
    def get_last_lr(self):
        return [0.05]


def test_lossless_training_matches_dense_bit_for_bit():
    """Reference idiom (examples/training/train_clm.py:641-653): SGD applied from
    post-accumulate hooks; with 7 kept bits the compressed run must equal the
    dense bf16 run exactly, step after step."""
    import neuzip_amd

    dense = _toy(3).cuda()
    comp = _toy(3)
    mgr = neuzip_amd.Manager(precision=7)
    mgr.convert(comp)
    comp = comp.cuda()
    sched = _Sched()
    for p in dense.parameters():
        p.register_post_accumulate_grad_hook(partial(neuzip_amd.lomo_hook, sched))
    for p in comp.parameters():
        hook = neuzip_amd.compressed_lomo_hook if isinstance(p, neuzip_amd.nn.Parameter) else neuzip_amd.lomo_hook
        p.register_post_accumulate_grad_hook(partial(hook, sched))
    torch.manual_seed(7)
    for step in range(5):
        x = torch.randn(16, 64, device="cuda", dtype=torch.bfloat16)
        l1 = dense(x).float().pow(2).mean()
        l2 = comp(x).float().pow(2).mean()
        assert torch.equal(l1, l2), step
        l1.backward()
        l2.backward()
        assert torch.equal(comp[0].weight(), dense[0].weight.data), step
        assert torch.equal(comp[2].weight(), dense[2].weight.data), step
        assert torch.equal(comp[0].bias.data, dense[0].bias.data)
    mgr._be.check()


def test_lossy_update_equals_reconstruction_of_update(oracle):
    import neuzip_amd

    mgr = neuzip_amd.Manager(precision=3)
    lin = torch.nn.Linear(96, 80, bias=False).to(torch.bfloat16)
    lin.weight.data.normal_(0, 0.02)
    m = torch.nn.Sequential(lin)
    mgr.convert(m)
    m = m.cuda()
    p = m[0].weight
    w0 = p()
    p._gradient = torch.randn(80, 96, device="cuda", dtype=torch.bfloat16)
    want = w0.clone().add_(p._gradient, alpha=-0.05)
    neuzip_amd.compressed_lomo_hook(_Sched(), p)
    got = p()
    assert np.array_equal(bits_of(got), closed_form_recon(bits_of(want), 3))


def test_side_stream_write_and_read():
    import neuzip_amd

    mgr = neuzip_amd.Manager()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        w = (torch.randn(2048, 512, device="cuda") * 0.02).to(torch.bfloat16)  # produced on `side`
        h = mgr.write(w)  # codec kernels are ordered behind the producer on the same stream
        out = mgr.read(h)
        assert torch.equal(out, w)
    side.synchronize()


def test_dummy_backend():
    import neuzip_amd

    mgr = neuzip_amd.Manager(algorithm=neuzip_amd.Algorithm.dummy)
    w = torch.randn(4, 8).to(torch.bfloat16)
    h = mgr.write(w)
    assert mgr.size(h) == 64 and torch.equal(mgr.read(h).cpu(), w)
    x = torch.randn(3, 8, device="cuda", dtype=torch.bfloat16)
    assert torch.equal(mgr.linear(h, x), torch.nn.functional.linear(x, w.cuda()))


class _Block(torch.nn.Module):
    def __init__(self, d, i):
        super().__init__()
        self.a = torch.nn.Linear(d, 2 * d, bias=(i % 2 == 0))
        self.b = torch.nn.Linear(2 * d, d, bias=False)
        self.c = torch.nn.Linear(d, d, bias=True)

    def forward(self, x):
        return x + self.c(self.b(torch.nn.functional.gelu(self.a(x))))


class _Stack(torch.nn.Module):
    def __init__(self, d, depth):
        super().__init__()
        self.inp = torch.nn.Linear(d, d)
        self.blocks = torch.nn.ModuleList([_Block(d, i) for i in range(depth)])

    def forward(self, x):
        x = self.inp(x)
        for b in self.blocks:
            x = b(x)
        return x


@pytest.mark.parametrize("depth", [1, 2, 5])
def test_decompress_ahead_matches_plain_forward(depth):
    import neuzip_amd

    torch.manual_seed(5)
    model = _Stack(256, depth).to(torch.bfloat16)
    for p in model.parameters():
        p.data.normal_(0, 0.02)
    mgr = neuzip_amd.Manager()
    mgr.convert(model)
    model = model.cuda()
    x = torch.randn(3, 256, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        want = model(x)
        for ahead, wrap in ((False, True), (True, True), (True, False)):
            print(f"case depth={depth} ahead={ahead} wrap={wrap}", flush=True)
            da = neuzip_amd.DecompressAhead(mgr, model, ahead=ahead, wrap=wrap)
            with da:
                for _ in range(3):  # with wrap the last block prefetches the first
                    got = model(x)
                    assert torch.equal(got, want)
            assert torch.equal(model(x), want)  # hook removed again
    mgr._be.check()


def test_decompress_ahead_sees_rewritten_weights():
    import neuzip_amd

    torch.manual_seed(6)
    model = _Stack(128, 2).to(torch.bfloat16)
    mgr = neuzip_amd.Manager()
    mgr.convert(model)
    model = model.cuda()
    x = torch.randn(2, 128, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad(), neuzip_amd.DecompressAhead(mgr, model) as da:
        y0 = model(x)
        lin = model.blocks[0].a
        mgr.write(lin.weight() * 2, lin.weight._handle)  # bumps the handle's write count
        y1 = model(x)
    with torch.no_grad():
        assert torch.equal(y1, model(x))
    assert not torch.equal(y0, y1)


def test_decompress_ahead_decodes_only_the_rewritten_tensor_again():
    """One write per parameter while the blocks are walked (the reference's
    in-backward update idiom, neuzip/utils.py:36-50): each write makes only that
    tensor decode again, the block's other tensors and the decode-ahead of the
    neighbouring block stay valid."""
    import neuzip_amd

    torch.manual_seed(8)
    model = _Stack(128, 3).to(torch.bfloat16)
    mgr = neuzip_amd.Manager()
    mgr.convert(model)
    model = model.cuda()
    x = torch.randn(2, 128, device="cuda", dtype=torch.bfloat16)
    calls = []
    real = mgr._be.read_batch

    def counting(plan, outs):
        calls.append(plan[2])
        return real(plan, outs)

    mgr._be.read_batch = counting
    try:
        # (blocks this small would share one launch: keep them apart, the test is about blocks)
        with torch.no_grad(), neuzip_amd.DecompressAhead(mgr, model, merge_small=False) as da:
            model(x)
            calls.clear()
            model(x)
            assert calls == [3, 3, 3]                   # steady state: one decode-ahead of three tensors per block
            halves = [(lin.weight._handle, lin.weight() * 0.5) for lin in
                      (model.blocks[0].a, model.blocks[0].b, model.blocks[0].c)]
            model(x)                                    # leaves block 0 decoded ahead for the next pass
            calls.clear()
            for h, t in halves:                         # one write per parameter of that block
                mgr.write(t, h)
            y = model(x)
            # its three tensors again, one at a time as each is used; the other blocks' decode-aheads as before
            assert sorted(calls) == [1, 1, 1, 3, 3, 3]
        with torch.no_grad():
            assert torch.equal(y, model(x))
    finally:
        del mgr._be.read_batch
    mgr._be.check()


def test_decode_under_graph_capture_replays_exactly():
    """The decode launches (per Linear, per block, per block with the side
    stream) captured into a HIP graph: every replay, with eager work and host
    synchronisation in between, gives the eager result for its input."""
    import neuzip_amd

    torch.manual_seed(7)
    model = _Stack(256, 4).to(torch.bfloat16)
    for p in model.parameters():
        p.data.normal_(0, 0.02)
    mgr = neuzip_amd.Manager()
    mgr.convert(model)
    model = model.cuda()
    xs = [torch.randn(1, 256, device="cuda", dtype=torch.bfloat16) for _ in range(5)]
    x_static = torch.zeros_like(xs[0])
    with torch.no_grad():
        wants = [model(x) for x in xs]
        for mode in ("per_linear", "per_block", "per_block_ahead"):
            print(f"case graph {mode}", flush=True)
            da = None if mode == "per_linear" else neuzip_amd.DecompressAhead(
                mgr, model, ahead=(mode == "per_block_ahead"), wrap=False)
            if da:
                da.enable()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                model(x_static)
                if da:
                    da.join()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                y_static = model(x_static)
                if da:
                    da.join()
            for x, want in zip(xs, wants):
                x_static.copy_(x)
                g.replay()
                got = y_static.clone()
                torch.cuda.synchronize()
                assert torch.equal(got, want)
                (x * 2).sum().item()  # eager work between replays
            if da:
                da.disable()
            del g
    mgr._be.check()


@pytest.mark.parametrize("ahead", [False, True])
def test_training_with_block_decode_equals_plain_training(ahead):
    """Forward and backward served from per-block decodes (the backward walks the
    blocks in reverse and re-compresses from hooks while it runs): same losses
    and weights as the per-Linear path, step after step."""
    import neuzip_amd

    def build():
        torch.manual_seed(21)
        m = _Stack(128, 3).to(torch.bfloat16)
        mgr = neuzip_amd.Manager(precision=7)
        mgr.convert(m)
        m = m.cuda()
        sched = _Sched()
        for p in m.parameters():
            hook = neuzip_amd.compressed_lomo_hook if isinstance(p, neuzip_amd.nn.Parameter) else neuzip_amd.lomo_hook
            p.register_post_accumulate_grad_hook(partial(hook, sched))
        return mgr, m

    mgr_a, plain = build()
    mgr_b, blocked = build()
    da = neuzip_amd.DecompressAhead(mgr_b, blocked, ahead=ahead)
    torch.manual_seed(8)
    with da:
        for step in range(4):
            x = torch.randn(8, 128, device="cuda", dtype=torch.bfloat16)
            l1 = plain(x).float().pow(2).mean()
            l2 = blocked(x).float().pow(2).mean()
            assert torch.equal(l1, l2), step
            l1.backward()
            l2.backward()
            for pa, pb in zip(plain.parameters(), blocked.parameters()):
                if isinstance(pa, neuzip_amd.nn.Parameter):
                    assert torch.equal(pa(), pb()), step
                else:
                    assert torch.equal(pa.data, pb.data), step
    mgr_a._be.check()
    mgr_b._be.check()


def test_read_batch_equals_single_reads(oracle):
    """One launch for several stored tensors, of different sizes and (auto mode)
    different segment geometries, gives what the single reads give."""
    import neuzip_amd

    for lane in (0, "auto"):
        mgr = neuzip_amd.Manager(lane_symbols=lane)
        sizes = [1, 4096, 65536 * 3 + 17, 1 << 20, 300_001, 65536, 8, 2_000_000] + [70_001 + i for i in range(12)]
        ws = [from_bits(stress_bits(1, n, seed=n % 89) if i % 2 else bf16_bits_normal(n, seed=i), (n,))
              for i, n in enumerate(sizes)]
        hs = [mgr.write(w) for w in ws]
        be = mgr._be
        print(f"case batch lane={lane}", flush=True)
        plan = be.batch_plan(hs)  # 20 tensors: more than one launch's worth of arguments
        outs = [torch.zeros((n + 7) & ~7, dtype=torch.bfloat16, device="cuda") for n in sizes]
        be.read_batch(plan, outs)
        for w, o, n in zip(ws, outs, sizes):
            assert torch.equal(o[:n].view(torch.int16), w.view(torch.int16))
        be.check()
        # a rejected argument decodes nothing
        import ctypes

        outs2 = [torch.zeros_like(o) for o in outs[:4]]
        names = (ctypes.c_char_p * 4)(*[h.encode() for h in hs[:3]], b"no such handle")
        ptrs = (ctypes.c_void_p * 4)(*[o.data_ptr() for o in outs2])
        caps = (ctypes.c_uint64 * 4)(*[o.numel() for o in outs2])
        rc = be._L.nz_manager_read_batch(be._h, names, ptrs, caps, 4, torch.cuda.current_stream().cuda_stream)
        assert rc != 0
        torch.cuda.synchronize()
        assert all(int(o.view(torch.int16).abs().max()) == 0 for o in outs2)


def _est_ratio(n, chunk, lane):
    """nz_api.hip's estimate of a tensor's stored exponent bytes over their entropy"""
    seg = 64 * lane
    full, rest = divmod(n, chunk)
    segs = full * -(-chunk // seg) + -(-rest // seg)
    return 1.0008 + (134.4 * segs + 78.0 * (full + (rest > 0)) + 600.0) / n


def _in_budget(n, chunk, lane, budget):
    return _est_ratio(n, chunk, lane) + 0.0003 <= budget


def _default_geometry(n, budget=1.01):
    """eight segments per chunk, the shortest from 256 symbols per lane up inside
    the budget; a tensor too small for any keeps 131072 / 256"""
    for lane in range(256, 513, 8):
        if _in_budget(n, 512 * lane, lane, budget):
            return 512 * lane, lane
    return 131072, 256


def _auto_geometry(n, cus=256, budget=1.01):
    """The per-tensor rule of nz_manager_create(lane_syms = NZ_LANE_SYMS_AUTO) with
    the library's own chunk: the default geometry of the tensor, unless one of
    k = 1, 2, 3 workgroups per compute unit (eight segments of 64..512 symbols
    per lane) is inside the size budget and modelled 10 % faster; a tensor too
    small for that gets 32 Ki chunks if the budget allows those."""
    dchunk, dlane = _default_geometry(n, budget)
    chunks = -(-n // dchunk)
    if chunks > 3 * cus:
        return dchunk, dlane
    step = (107, 147, 215)
    best_t, best = dlane * step[max(1, -(-chunks // cus)) - 1], None
    for k in (1, 2, 3):
        lane = -(-(-(-n // (k * cus * 512))) // 8) * 8
        if lane < 64 or lane > 512 or not _in_budget(n, 512 * lane, lane, budget):
            continue
        t = lane * step[k - 1]
        if 10 * t < 9 * best_t:
            best_t, best = t, lane
    if best:
        return 512 * best, best
    if n < 64 * cus * 512 and _in_budget(n, 32768, 64, budget):
        return 32768, 64
    return dchunk, dlane


def test_auto_lane_symbols(oracle):
    """Per-tensor geometry inside the size budget: at the default budget every
    tensor keeps the default geometry or gets longer segments, and what is
    stored for the exponents of a tensor of a million elements or more stays
    within 1.01 x their order-0 entropy; a caller who raises the budget gets
    the shorter segments that let a small tensor fill the device.  The stored
    bytes are those of the oracle at the chosen geometry, reads are exact."""
    import neuzip_amd

    assert _default_geometry(14336 * 4096) == (131072, 256) and _default_geometry(4096 * 4096) == (131072, 256)
    assert _default_geometry(4096 * 1024) == (135168, 264) and _default_geometry(1024 * 1024) == (143360, 280)
    assert _default_geometry(40_001) == (131072, 256)  # too small for any geometry to reach the budget
    assert _auto_geometry(14336 * 4096) == (131072, 256) and _auto_geometry(4096 * 4096) == (131072, 256)
    assert _auto_geometry(14336 * 4096, budget=1.05) == (114688, 224)
    assert _auto_geometry(4096 * 4096, budget=1.05) == (32768, 64)
    assert _auto_geometry(16384 * 4096, budget=1.05) == (131072, 256)
    sizes = (1000, 40_001, 1 << 20, 25_165_824, 40_000_000, 14336 * 4096, 70_000_000, 110_000_000)
    for kwargs, cases in (
        (dict(lane_symbols="auto"), tuple((n,) + _auto_geometry(n) for n in sizes)),
        (dict(lane_symbols="auto", size_budget=1.05), tuple((n,) + _auto_geometry(n, budget=1.05) for n in sizes)),
        (dict(chunk_size=65536, lane_symbols="auto"), ((1 << 20, 65536, 344), (40_000_000, 65536, 344))),
        (dict(chunk_size=65536, lane_symbols="auto", size_budget=1.05),
         ((1 << 20, 65536, 128), (40_000_000, 65536, 256), (70_000_000, 65536, 256))),
    ):
        mgr = neuzip_amd.Manager(**kwargs)
        for n, chunk, lane in cases:
            print(f"case auto {kwargs} n={n}", flush=True)
            w = from_bits(bf16_bits_normal(n, seed=n % 97), (n,))
            h = mgr.write(w)
            assert mgr._be.geometry(h) == (chunk, lane)
            o_comp, o_packed = oracle.compress_bf16(bits_of(w), 7, chunk, lane, threads=8)
            assert mgr.size(h) == o_comp.size + o_packed.size
            assert torch.equal(mgr.read(h), w)
            if n >= 1 << 20 and "size_budget" not in kwargs:
                exps = ((bits_of(w) >> 7) & 0xFF).astype(np.uint8)
                assert mgr.size(h) - n <= 1.01 * chunk_entropy_bytes(exps), (n, chunk, lane)
            del w
        mgr._be.check()


def test_trim_releases_the_write_scratch():
    """After trim the manager holds little more than the compressed bytes."""
    import neuzip_amd

    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    mgr = neuzip_amd.Manager()
    n = 32 * 1024 * 1024
    w = from_bits(bf16_bits_normal(n, seed=4), (n,))
    free0 = torch.cuda.mem_get_info()[0]
    h = mgr.write(w)
    held_with_scratch = free0 - torch.cuda.mem_get_info()[0]
    mgr.trim()
    held = free0 - torch.cuda.mem_get_info()[0]
    stored = mgr.size(h)
    assert held_with_scratch > 2 * stored           # the encode workspace dominates
    assert stored <= held <= stored + (64 << 20)    # allocator granularity aside
    assert torch.equal(mgr.read(h), w)              # reads need no scratch
    mgr.write(w * 2, h)                             # and a write brings it back
    assert torch.equal(mgr.read(h), w * 2)
    mgr._be.check()


def test_write_many_equals_single_writes(oracle):
    import neuzip_amd

    for lane in (0, "auto"):
        one, many = neuzip_amd.Manager(lane_symbols=lane), neuzip_amd.Manager(lane_symbols=lane)
        sizes = [(64, 1000), (3,), (0,), (300_000,), (1 << 20,)] + [(1000 + i,) for i in range(14)]  # 19 tensors
        ws = [from_bits(bf16_bits_normal(int(np.prod(s)), seed=i), s) for i, s in enumerate(sizes)]
        hs = [f"w{i}" for i in range(len(ws))]
        many.write(ws[3], hs[0])  # replaced by the batch
        for w, h in zip(ws, hs):
            one.write(w, h)
        many.write_many(ws, hs)
        for w, h in zip(ws, hs):
            assert many.size(h) == one.size(h)
            assert torch.equal(many.read(h), w) and many.read(h).shape == w.shape
        a, b = one._be.export(hs[4]), many._be.export(hs[4])
        assert all(torch.equal(x, y) for x, y in zip(a, b))
        with pytest.raises(ValueError):
            many.write_many(ws[:2], ["same", "same"])
        many._be.check()


@pytest.mark.parametrize("behind", [True, False])
def test_rewrite_in_place_needs_no_size_round_trip(oracle, behind):
    """Writing again under handles that hold tensors of the same size (the
    re-compress after an optimizer step, neuzip/__init__.py:25-35) goes straight
    into the entries' buffers; the stored bytes are still the oracle's, and an
    entry whose container outgrows its buffer is re-placed without losing data."""
    import neuzip_amd

    mgr = neuzip_amd.Manager()
    mgr.write_behind = behind  # single writes of small tensors wait for each other and share a launch, or do not
    shapes = [(300, 1000), (257, 513), (64, 4096)]
    ws = [from_bits(bf16_bits_normal(int(np.prod(s)), seed=i), s) for i, s in enumerate(shapes)]
    hs = [mgr.write(w) for w in ws]
    assert mgr._be.rewrite_stats() == (0, 0)
    # three optimizer-like steps over all tensors (slots alternate), single writes and batches
    for step in range(3):
        ws = [(w.float() * (1.0 + 0.001 * (step + 1))).to(torch.bfloat16) for w in ws]
        if step == 1:
            for w, h in zip(ws, hs):
                mgr.write(w, h)
        else:
            mgr.write_many(ws, hs)
        for w, h in zip(ws, hs):
            assert torch.equal(mgr.read(h), w)
            o_comp, o_packed = oracle.compress_bf16(bits_of(w), 7, *mgr._be.geometry(h))
            assert mgr.size(h) == o_comp.size + o_packed.size
            comp, packed, _ = mgr._be.export(h)
            assert np.array_equal(comp.numpy(), o_comp) and np.array_equal(packed.numpy(), o_packed)
    batches, outgrown = mgr._be.rewrite_stats()
    assert batches == (3 if behind else 2 + len(hs)) and outgrown == 0
    # a handle whose new content compresses far worse than the old: the container
    # outgrows the buffer it has and moves to a larger one
    n = 1 << 20
    flat = torch.full((n,), 0.5, dtype=torch.bfloat16, device="cuda")     # one exponent value: a tiny container
    h = mgr.write(flat)
    small, small_container = mgr.size(h), mgr._be.exp_bytes(h)
    noisy = from_bits(stress_bits(1024, 1024, seed=3), (n,))
    mgr.write(noisy, h)
    assert torch.equal(mgr.read(h).view(torch.int16), noisy.view(torch.int16))
    assert mgr._be.exp_bytes(h) > 20 * small_container
    assert mgr._be.rewrite_stats() == (batches + 1, 1)
    mgr.write(flat, h)                                                    # and back: fits the larger buffer
    assert torch.equal(mgr.read(h), flat) and mgr.size(h) == small
    assert mgr._be.rewrite_stats() == (batches + 2, 1)
    # a different element count under the same handle takes the sized-to-fit route
    mgr.write(flat[: n // 2], h)
    assert torch.equal(mgr.read(h), flat[: n // 2])
    assert mgr._be.rewrite_stats() == (batches + 2, 1)
    mgr._be.check()


def test_records_are_placed_again_when_a_workgroup_gives_up_waiting(oracle):
    """The encode kernel places its records itself; a workgroup waits for the
    record sizes of the chunks before its own, and gives up after a bounded
    number of looks.  With that number forced to zero from the host, workgroups
    whose predecessors are not done at their first look give up (every kernel
    still runs to its end): the records are then placed by the second kernel,
    at once in nz_encode, at the next use in a manager, and the stored bytes
    are the oracle's either way."""
    import neuzip_amd
    from neuzip_amd import _lib
    from test_gpu_parity import gpu_encode

    L = _lib.load()
    n = 40 * 131072 + 777                       # 41 chunks
    bits = bf16_bits_normal(n, seed=21)
    o_comp, o_packed = oracle.compress_bf16(bits, 7, 131072, 256)
    mgr = neuzip_amd.Manager(lane_symbols=256)
    w = from_bits(bits, (n,))
    h = mgr.write(w)                            # sized to fit: the two-kernel route
    try:
        L.nz_set_lookback_spins(0)
        print("case stateless encode, spin limit 0", flush=True)
        comp, packed = gpu_encode(bits, 7)
        assert np.array_equal(comp.cpu().numpy(), o_comp) and np.array_equal(packed.cpu().numpy(), o_packed)
        print("case in-place rewrites, spin limit 0", flush=True)
        w2 = (w.float() * 1.001).to(torch.bfloat16)
        o2_comp, o2_packed = oracle.compress_bf16(bits_of(w2), 7, 131072, 256)
        for _ in range(3):
            mgr.write(w2, h)
            assert torch.equal(mgr.read(h), w2)
            comp, packed, _ = mgr._be.export(h)
            assert np.array_equal(comp.numpy(), o2_comp) and np.array_equal(packed.numpy(), o2_packed)
        again = mgr._be.placed_again()
        print(f"placed again: {again} of 3", flush=True)
    finally:
        L.nz_set_lookback_spins(1 << 21)
    for _ in range(2):                          # a scratch in which a workgroup gave up is marked: the next encode
        mgr.write(w2, h)                        # that uses it (one per rewrite slot) leaves the placing to the second
        assert torch.equal(mgr.read(h), w2)     # kernel once more and takes the mark away
    before = mgr._be.placed_again()
    mgr.write(w, h)                             # with the usual bound nothing gives up
    assert torch.equal(mgr.read(h), w)
    comp, packed, _ = mgr._be.export(h)
    assert np.array_equal(comp.numpy(), o_comp) and np.array_equal(packed.numpy(), o_packed)
    assert mgr._be.placed_again() == before
    mgr._be.check()


def test_in_place_rewrites_of_two_managers_on_two_streams(oracle):
    """Two managers re-compress their tensors at the same time on streams of
    their own (encode kernels of both are resident together; each places its own
    records): every read returns what was written last."""
    import neuzip_amd

    n = 24 * 131072 + 5
    mgrs = [neuzip_amd.Manager(), neuzip_amd.Manager(precision=3)]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]  # default priority
    base = [from_bits(bf16_bits_normal(n, seed=40 + i), (n,)) for i in range(2)]
    hs = [m.write(w) for m, w in zip(mgrs, base)]
    torch.cuda.synchronize()
    last = [None, None]
    for it in range(12):
        for i in (0, 1):
            with torch.cuda.stream(streams[i]):
                w = (base[i].float() * (1.0 + 0.002 * (it + 1))).to(torch.bfloat16)
                mgrs[i].write(w, hs[i])
                last[i] = w
    for i in (0, 1):
        with torch.cuda.stream(streams[i]):
            got = mgrs[i].read(hs[i])
            want = from_bits(oracle.reconstruct(bits_of(last[i]), 7 if i == 0 else 3), (n,))
        streams[i].synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        assert mgrs[i]._be.placed_again() == 0
        mgrs[i]._be.check()


def test_small_writes_are_held_back_and_no_call_can_tell(oracle):
    """Writes of small tensors wait, as copies made at the time of the call, until
    16 of them (or enough elements to fill the device) share one encode launch;
    every other call on the manager stores them first.  What is stored is what
    the tensor held when ``write`` was called, byte for byte the oracle's."""
    import neuzip_amd

    mgr = neuzip_amd.Manager()
    be = mgr._be
    n = 200_000
    ws = [from_bits(bf16_bits_normal(n, seed=40 + i), (n,)) for i in range(20)]

    # the value at the time of the call counts, whatever happens to the tensor afterwards
    src = ws[0].clone()
    h = mgr.write(src)
    assert [w[0] for w in be._held] == [h]
    src.zero_()
    del src
    assert torch.equal(mgr.read(h), ws[0]) and not be._held
    # two writes under one handle before anything is stored: the later one is what is kept
    mgr.write(ws[1], h)
    mgr.write(ws[2], h)
    assert [w[0] for w in be._held] == [h] and torch.equal(be._held[0][1], ws[2])
    assert mgr.size(h) > 0 and not be._held  # size() looks at the store: stored first
    o_comp, o_packed = oracle.compress_bf16(bits_of(ws[2]), 7, *be.geometry(h))
    comp, packed, _ = be.export(h)
    assert np.array_equal(comp.numpy(), o_comp) and np.array_equal(packed.numpy(), o_packed)
    # the sixteenth write stores all sixteen with one launch
    before = be.rewrite_stats()
    hs = []
    for i in range(15):
        hs.append(mgr.write(ws[i]))
        assert len(be._held) == i + 1
    hs.append(mgr.write(ws[15]))
    assert not be._held
    for i, hh in enumerate(hs):
        assert torch.equal(mgr.read(hh), ws[i]), i
    # ... and again into the buffers the entries have: one batch in place
    for i, hh in enumerate(hs):
        mgr.write(ws[i + 4], hh)
    assert not be._held
    assert be.rewrite_stats()[0] == before[0] + 1
    for i, hh in enumerate(hs):
        assert torch.equal(mgr.read(hh), ws[i + 4]), i
    # explicit flush; a tensor too large to be worth a copy is stored at once
    mgr.write(ws[0], hs[0])
    assert be._held
    mgr.flush()
    assert not be._held and torch.equal(mgr.read(hs[0]), ws[0])
    big = from_bits(bf16_bits_normal(be.ahead_fill // 4 + 8, seed=3), (be.ahead_fill // 4 + 8,))
    hb = mgr.write(big)
    assert not be._held and torch.equal(mgr.read(hb), big)
    # written on one stream, stored by a call on another
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fresh = (ws[5].float() * 1.25).to(torch.bfloat16)
        mgr.write(fresh, hs[1])
        del fresh
    assert be._held
    got = mgr.read(hs[1])
    assert torch.equal(got, (ws[5].float() * 1.25).to(torch.bfloat16))
    torch.cuda.current_stream().wait_stream(side)
    # a call that cannot store them (its stream is being captured) is refused and nothing is lost
    mgr.write(ws[7], hs[2])
    out = torch.empty(ws[7].numel(), dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        with pytest.raises(ValueError, match="being captured"):
            be.read_into(hs[2], out)
        out.add_(0)
    assert [w[0] for w in be._held] == [hs[2]]
    assert torch.equal(mgr.read(hs[2]), ws[7]) and not be._held
    # switched off: every write is stored by its own call
    mgr.write(ws[8], hs[3])
    mgr.write_behind = False
    assert not be._held and torch.equal(mgr.read(hs[3]), ws[8])
    mgr.write(ws[9], hs[3])
    assert not be._held and torch.equal(mgr.read(hs[3]), ws[9])
    be.check()


def test_the_references_update_loop_reads_ahead_and_writes_behind():
    """The reference's training example updates every compressed parameter with
    ``write(read(handle).add_(gradient, alpha=-lr), handle)`` (examples/training/
    train_clm.py:822-833).  Served with weights decoded ahead and writes held
    back, the loop leaves exactly the weights that plain dense SGD leaves."""
    import neuzip_amd

    torch.manual_seed(11)
    shapes = [(256, 512), (512, 512), (128, 1024), (1024, 256)] * 5
    dense = [(torch.randn(s, device="cuda") * 0.02).to(torch.bfloat16) for s in shapes]
    mgr = neuzip_amd.Manager(precision=7)
    hs = [mgr.write(w) for w in dense]
    lr = 1e-2
    for step in range(4):
        grads = [(torch.randn(s, device="cuda") * 0.01).to(torch.bfloat16) for s in shapes]
        for h, g in zip(hs, grads):
            mgr.write(mgr.read(h).add_(g, alpha=-lr), h)
        for w, g in zip(dense, grads):
            w.add_(g, alpha=-lr)
        if step % 2:  # looked at after some steps only: the next step may start with writes still held
            for h, w in zip(hs, dense):
                assert torch.equal(mgr.read(h), w), step
    hits, waste = mgr._be.ahead_stats()
    assert hits > 40, (hits, waste)
    for h, w in zip(hs, dense):
        assert torch.equal(mgr.read(h), w)
    mgr._be.check()


def test_lomo_hooks_with_weights_decoded_ahead_and_writes_held_back():
    """The reference's memory-efficient training (neuzip/__init__.py:25-35): every
    compressed parameter is updated and written back from a hook in the middle
    of the backward pass, so a weight is asked for twice in a row (backward, then
    update) and written while the weights of the layers before it wait decoded.
    Equal, step after step, to the dense run and to a manager that decodes and
    stores every tensor on its own."""
    import neuzip_amd

    def deep(seed):
        torch.manual_seed(seed)
        layers = []
        for k in range(8):
            layers += [torch.nn.Linear(256, 256, bias=(k % 3 == 0)), torch.nn.GELU()]
        m = torch.nn.Sequential(*layers[:-1]).to(torch.bfloat16)
        for p in m.parameters():
            p.data.normal_(0, 0.05)
        return m

    sched = _Sched()
    dense = deep(5).cuda()
    models, mgrs = [], []
    for plain in (False, True):
        m = deep(5)
        mgr = neuzip_amd.Manager(precision=7)
        if plain:
            mgr.decode_ahead = False
            mgr.write_behind = False
        mgr.convert(m)
        models.append(m.cuda())
        mgrs.append(mgr)
    for p in dense.parameters():
        p.register_post_accumulate_grad_hook(partial(neuzip_amd.lomo_hook, sched))
    for m in models:
        for p in m.parameters():
            hook = neuzip_amd.compressed_lomo_hook if isinstance(p, neuzip_amd.nn.Parameter) else neuzip_amd.lomo_hook
            p.register_post_accumulate_grad_hook(partial(hook, sched))
    torch.manual_seed(9)
    for step in range(6):
        x = torch.randn(32, 256, device="cuda", dtype=torch.bfloat16)
        losses = [m(x).float().pow(2).mean() for m in [dense] + models]
        assert torch.equal(losses[0], losses[1]) and torch.equal(losses[1], losses[2]), step
        for l in losses:
            l.backward()
        if step % 2:
            for k in range(0, 15, 2):
                assert torch.equal(models[0][k].weight(), dense[k].weight.data), (step, k)
                assert torch.equal(models[1][k].weight(), dense[k].weight.data), (step, k)
    hits, waste = mgrs[0]._be.ahead_stats()
    assert hits > 30 and waste < hits // 2, (hits, waste)
    assert mgrs[1]._be.ahead_stats() == (0, 0)
    for mgr in mgrs:
        mgr._be.check()
