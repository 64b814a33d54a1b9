"""Row gather on a stored table and the compressed Embedding module."""
import numpy as np
import pytest

from conftest import bf16_bits_normal, stress_bits

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _table_bits(rows, dim, seed, kind="normal"):
    bits = bf16_bits_normal(rows * dim, seed) if kind == "normal" else stress_bits(rows, dim, seed)
    return np.where((bits & 0x7F80) == 0x7F80, np.uint16(0x3F80), bits).astype(np.uint16)


def _dev(bits, rows, dim):
    return torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16).view(rows, dim)


def _table(rows, dim, seed, kind="normal"):
    return _dev(_table_bits(rows, dim, seed, kind), rows, dim)


@pytest.mark.parametrize("rows,dim,precision,norm,lane", [
    (1000, 64, 7, 0, 0),        # many rows per chunk
    (300, 4096, 7, 0, 0),       # 16 rows per chunk
    (37, 100_000, 7, 0, 0),     # a row spans several chunks and starts anywhere inside one
    (513, 768, 3, 512, "auto"),
    (129, 40, 0, 8, 128),       # odd row length: rows straddle groups of 8
])
def test_gather_rows_equals_oracle_rows(oracle, rows, dim, precision, norm, lane):
    """Gathered rows against the CPU oracle's reconstruction of the same bits
    (what the reference's Embedding.forward indexes after decompressing the
    whole table, neuzip/nn/embedding.py:30-39), and against the full read."""
    import neuzip_amd

    mgr = neuzip_amd.Manager(precision=precision, normalizer_size=norm, lane_symbols=lane)
    bits = _table_bits(rows, dim, seed=rows, kind="stress" if norm else "normal")
    h = mgr.write(_dev(bits, rows, dim))
    want = oracle.reconstruct_normalized(bits, precision, norm) if norm else oracle.reconstruct(bits, precision)
    full = _dev(want, rows, dim)
    assert torch.equal(mgr.read(h), full)
    g = torch.Generator().manual_seed(rows)
    for count in (1, 7, 200):
        idx = torch.randint(0, rows, (count,), generator=g)
        idx[0], idx[-1] = rows - 1, 0
        print(f"case gather rows={rows} dim={dim} count={count}", flush=True)
        got = mgr.gather_rows(h, idx.cuda())
        assert got.shape == (count, dim)
        assert torch.equal(got, full[idx.cuda()])
    mgr._be.check()
    # an index outside the table: zeros, and the manager reports it
    got = mgr.gather_rows(h, torch.tensor([0, rows, -1, 1]).cuda())
    assert torch.equal(got[0], full[0]) and torch.equal(got[3], full[1])
    assert int(got[1].view(torch.int16).abs().max()) == 0 and int(got[2].view(torch.int16).abs().max()) == 0
    with pytest.raises(RuntimeError, match="outside the table"):
        mgr._be.check()


def test_embedding_module_and_unroll_convert():
    import neuzip_amd
    from neuzip_amd.utils import _unroll_convert

    torch.manual_seed(3)

    class Tiny(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = torch.nn.Embedding(500, 128, padding_idx=0)
            self.blocks = torch.nn.ModuleList([torch.nn.Linear(128, 128) for _ in range(2)])
            self.lm_head = torch.nn.Linear(128, 500, bias=False)

        def forward(self, ids):
            x = self.emb(ids)
            for b in self.blocks:
                x = torch.relu(b(x))
            return self.lm_head(x)

    dense = Tiny().to(torch.bfloat16).cuda()
    ids = torch.randint(0, 500, (3, 17), device="cuda")
    with torch.no_grad():
        want = dense(ids)
    mgr = neuzip_amd.Manager()
    model = _unroll_convert(mgr, dense)
    assert isinstance(model.emb, neuzip_amd.nn.Embedding) and repr(model.emb).startswith("Embedding(!")
    assert isinstance(model.lm_head, neuzip_amd.nn.Linear)  # unlike convert(), nothing is skipped
    assert all(isinstance(b, neuzip_amd.nn.Linear) for b in model.blocks)
    assert model.emb.weight.numel() == 0 and mgr.size(model.emb.weight._handle) > 0
    with torch.no_grad():
        assert torch.equal(model(ids), want)

    # max_norm goes through torch's own renormalisation
    e = torch.nn.Embedding(50, 64, max_norm=0.5).to(torch.bfloat16).cuda()
    w0 = e.weight.data.clone()
    ce = neuzip_amd.nn.Embedding(mgr, e)
    ids = torch.randint(0, 50, (9,), device="cuda")
    with torch.no_grad():
        ref = torch.nn.functional.embedding(ids, w0.clone(), None, 0.5, 2.0)
        assert torch.equal(ce(ids), ref)
    # the dummy backend keeps the module usable
    dm = neuzip_amd.Manager(algorithm=neuzip_amd.Algorithm.dummy)
    de = neuzip_amd.nn.Embedding(dm, torch.nn.Embedding(20, 8).to(torch.bfloat16).cuda())
    assert de(torch.tensor([[1, 2]]).cuda()).shape == (1, 2, 8)
    mgr._be.check()


def test_large_lookups_are_bounded(oracle):
    """A lookup of more rows than the table has chunks goes through one full
    read; a lookup whose slots would exceed the scratch cap is served in slices;
    more than 65535 rows are fine; all equal the oracle's rows."""
    import neuzip_amd

    rows, dim = 3000, 4096          # 94 chunks of 131072 elements, 32 rows per chunk
    bits = _table_bits(rows, dim, seed=5)
    mgr = neuzip_amd.Manager()
    h = mgr.write(_dev(bits, rows, dim))
    full = _dev(oracle.reconstruct(bits, 7), rows, dim)
    g = torch.Generator().manual_seed(1)
    assert mgr._be.geometry(h) == (131072, 256)
    for count in (50, 93, 94, 5000):                      # below / at / above the number of chunks
        idx = torch.randint(0, rows, (count,), generator=g).cuda()
        print(f"case lookup count={count}", flush=True)
        assert torch.equal(mgr.gather_rows(h, idx), full[idx])
    idx = torch.tensor([0, rows, -1, rows - 1] * 40).cuda()  # the full-read route zeroes rows outside the table too
    got = mgr.gather_rows(h, idx)
    assert torch.equal(got[0], full[0]) and torch.equal(got[3], full[rows - 1])
    assert int(got[1].view(torch.int16).abs().max()) == 0 and int(got[2].view(torch.int16).abs().max()) == 0
    with pytest.raises(RuntimeError, match="outside the table"):
        mgr._be.check()
    mgr._be.check()                 # reported once
    # the native gather in slices: 2500 rows of 2 chunk-sized slots each are 1.3 GB of slots, the cap a quarter GiB
    rows2, dim2 = 70_000, 24        # rows straddle chunk boundaries (131072 is not a multiple of 24)
    bits2 = _table_bits(rows2, dim2, seed=6)
    h2 = mgr.write(_dev(bits2, rows2, dim2))
    full2 = _dev(oracle.reconstruct(bits2, 7), rows2, dim2)
    idx = torch.randint(0, rows2, (2500,), generator=g).cuda()
    got = mgr._be.gather_rows(h2, idx, dim2)
    assert torch.equal(got, full2[idx])
    many = torch.randint(0, rows2, (66_000,), generator=g).cuda()   # more rows than a grid dimension of 65535 holds
    assert torch.equal(mgr.gather_rows(h2, many), full2[many])
    assert torch.equal(mgr._be.gather_rows(h2, many[:66_000], dim2), full2[many])
    mgr._be.check()


def test_embedding_table_gets_short_segments_under_per_tensor_geometry(oracle):
    """With a manager that chooses the geometry per tensor and whose size budget
    allows it, a converted Embedding stores its table in 32 Ki chunks of eight
    4 Ki segments (a lookup decodes whole chunks); at the default budget the table
    keeps the geometry of its size.  The rows are the oracle's either way."""
    import neuzip_amd

    rows, dim = 5000, 1024          # 5.1 M elements: on its own the table would get longer segments
    bits = _table_bits(rows, dim, seed=9)
    emb = torch.nn.Embedding(rows, dim).to(torch.bfloat16)
    emb.weight.data = _dev(bits, rows, dim).cpu()
    full = _dev(oracle.reconstruct(bits, 7), rows, dim)
    idx = torch.randint(0, rows, (3, 17), generator=torch.Generator().manual_seed(2)).cuda()
    for budget, geometry in ((1.04, (32768, 64)), (None, (135168, 264))):
        mgr = neuzip_amd.Manager(lane_symbols="auto", size_budget=budget)
        conv = neuzip_amd.nn.Embedding(mgr, emb)
        h = conv.weight._handle
        assert mgr._be.geometry(h) == geometry
        assert torch.equal(conv(idx), full[idx])
        assert torch.equal(mgr.read(h).view(rows, dim), full)
        mgr._be.check()
