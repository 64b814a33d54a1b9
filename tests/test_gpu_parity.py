"""HIP path vs CPU oracle through the C ABI (needs an MI355X)."""
import ctypes

import numpy as np
import pytest

from conftest import bf16_bits_normal, chunk_entropy_bytes, closed_form_recon, stress_bits

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _lib():
    from neuzip_amd import _lib

    return _lib.load(), _lib


def _to_dev(bits: np.ndarray):
    return torch.from_numpy(bits.view(np.int16).copy()).cuda()


def gpu_encode(bits, s, chunk=131072, lane=256, norm_size=0):
    """-> (container, stored packed stream[, normalizer bytes when norm_size > 0]) as device tensors"""
    L, m = _lib()
    n = bits.size
    d_in = _to_dev(bits) if n else torch.empty(0, dtype=torch.int16, device="cuda")
    cap = L.nz_exp_bound_bytes(n, chunk, lane)
    assert cap > 0
    ws_bytes = L.nz_encode_workspace_bytes(n, chunk, lane)
    comp = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    packed = torch.zeros(max(8, L.nz_packed_stored_bytes(n, s, chunk, lane)), dtype=torch.uint8, device="cuda")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    aux = torch.zeros(4, dtype=torch.int64, device="cuda")
    total = ctypes.c_uint64(0)
    st = torch.cuda.current_stream().cuda_stream
    norm = torch.zeros(L.nz_norm_bytes(n, norm_size) + 8, dtype=torch.uint8, device="cuda")
    rc = L.nz_encode(d_in.data_ptr(), n, s, chunk, lane, packed.data_ptr(), comp.data_ptr(), cap,
                     ws.data_ptr(), ws_bytes, aux.data_ptr(), aux.data_ptr() + 8, ctypes.byref(total),
                     norm_size, norm.data_ptr(), st)
    assert rc == 0, m.last_error()
    torch.cuda.synchronize()
    res = comp[: total.value].clone(), packed[: L.nz_packed_stored_bytes(n, s, chunk, lane)].clone()
    return res + (norm[: L.nz_norm_bytes(n, norm_size)].clone(),) if norm_size else res


def gpu_decode(comp, packed, n, s, chunk=131072, lane=256, check=True, norm_size=0, norm=None):
    L, m = _lib()
    if norm_size:
        norm = torch.cat([norm, torch.zeros(8, dtype=torch.uint8, device="cuda")])
    out = torch.zeros(max(n, 8), dtype=torch.int16, device="cuda")
    status = torch.zeros(2, dtype=torch.int32, device="cuda")
    if packed.numel() < 8:
        packed = torch.cat([packed, torch.zeros(8, dtype=torch.uint8, device="cuda")])
    st = torch.cuda.current_stream().cuda_stream
    rc = L.nz_decode(comp.data_ptr(), comp.numel(), packed.data_ptr(), n, s, chunk, lane,
                     out.data_ptr(), status.data_ptr(), 1 if check else 0, norm_size,
                     norm.data_ptr() if norm_size else None, st)
    torch.cuda.synchronize()
    return rc, out[:n].cpu().numpy().view(np.uint16)


SIZES = [0, 1, 7, 8, 9, 511, 512, 513, 4095, 65535, 65536, 65537, 200_000, 1_000_003]


@pytest.mark.parametrize("s", [7, 3, 1, 0])
@pytest.mark.parametrize("n", SIZES)
def test_roundtrip_matches_oracle(oracle, n, s):
    bits = bf16_bits_normal(n, seed=n + s)
    print(f"case n={n} s={s}", flush=True)
    comp, packed = gpu_encode(bits, s)
    # container and packed stream are byte-identical to the oracle's
    o_comp, o_packed = oracle.compress_bf16(bits, s, 131072, 256)
    assert np.array_equal(packed.cpu().numpy(), o_packed)
    assert np.array_equal(comp.cpu().numpy(), o_comp)
    rc, out = gpu_decode(comp, packed, n, s)
    assert rc == 0
    assert np.array_equal(out, oracle.reconstruct(bits, s))
    assert np.array_equal(out, closed_form_recon(bits, s))


@pytest.mark.parametrize("lane,chunk", [(128, 65536), (256, 65536), (344, 65536), (352, 65536), (512, 65536),
                                        (1024, 65536), (1000, 65536), (16, 1024), (24, 2560), (64, 4096),
                                        (2048, 1 << 20), (256, 131072), (344, 131072), (2048, 131072),
                                        (512, 262144)])
def test_geometries(oracle, lane, chunk):
    n = 3 * chunk + 1234 if chunk <= 65536 else chunk + 777
    bits = bf16_bits_normal(n, seed=lane)
    print(f"case lane={lane} chunk={chunk} n={n}", flush=True)
    comp, packed = gpu_encode(bits, 7, chunk, lane)
    o_comp, _ = oracle.compress_bf16(bits, 7, chunk, lane)
    assert np.array_equal(comp.cpu().numpy(), o_comp)
    rc, out = gpu_decode(comp, packed, n, 7, chunk, lane)
    assert rc == 0 and np.array_equal(out, bits)


def test_all_bit_patterns(oracle):
    allv = np.arange(65536, dtype=np.uint16)
    bits = np.tile(allv, 3)
    for s in (7, 3, 1, 0):
        print(f"case all patterns s={s}", flush=True)
        comp, packed = gpu_encode(bits, s)
        rc, out = gpu_decode(comp, packed, bits.size, s)
        assert rc == 0
        assert np.array_equal(out, closed_form_recon(bits, s))
        assert np.array_equal(out, oracle.reconstruct(bits, s))


def test_cross_cpu_gpu(oracle):
    n = 300_000
    bits = stress_bits(300, 1000, seed=5)
    for s in (7, 3):
        print(f"case cross s={s}", flush=True)
        o_comp, o_packed = oracle.compress_bf16(bits, s, 65536, 512)
        rc, out = gpu_decode(torch.from_numpy(o_comp).cuda(), torch.from_numpy(o_packed).cuda(), n, s, 65536, 512)
        assert rc == 0 and np.array_equal(out, oracle.reconstruct(bits, s))
        comp, packed = gpu_encode(bits, s, 65536, 512)
        rc2, out2 = oracle.decompress_bf16(comp.cpu().numpy(), packed.cpu().numpy(), n, s)
        assert rc2 == 0 and np.array_equal(out2, oracle.reconstruct(bits, s))


def test_incompressible_goes_raw(oracle):
    rng = np.random.default_rng(3)
    n = 150_000
    bits = rng.integers(0, 65536, n).astype(np.uint16)
    print("case raw", flush=True)
    comp, packed = gpu_encode(bits, 7)
    o_comp, _ = oracle.compress_bf16(bits, 7, 131072, 256)
    assert np.array_equal(comp.cpu().numpy(), o_comp)
    L, _m = _lib()
    assert comp.numel() <= L.nz_exp_bound_bytes(n, 131072, 256)
    rc, out = gpu_decode(comp, packed, n, 7)
    assert rc == 0 and np.array_equal(out, bits)


def test_constant_and_two_symbol(oracle):
    for name, bits in (("zeros", np.zeros(70_000, np.uint16)),
                       ("const", np.full(70_000, 0x3C00, np.uint16)),
                       ("two", np.where(np.arange(70_000) % 97 == 0, 0x3C00, 0x0080).astype(np.uint16))):
        print(f"case {name}", flush=True)
        comp, packed = gpu_encode(bits, 7)
        o_comp, _ = oracle.compress_bf16(bits, 7, 131072, 256)
        assert np.array_equal(comp.cpu().numpy(), o_comp)
        rc, out = gpu_decode(comp, packed, bits.size, 7)
        assert rc == 0 and np.array_equal(out, bits)


def test_corrupt_container_is_reported(oracle):
    n = 100_000
    bits = bf16_bits_normal(n, seed=11)
    comp, packed = gpu_encode(bits, 7)
    bad = comp.clone()
    bad[bad.numel() // 2] ^= 0x5A  # flip bits inside the word stream
    print("case corrupt words", flush=True)
    rc, _ = gpu_decode(bad, packed, n, 7)
    assert rc == -6
    bad = comp.clone()
    bad[64:72] = 0xFF  # directory entries out of range
    print("case corrupt directory", flush=True)
    rc, _ = gpu_decode(bad, packed, n, 7)
    assert rc == -6


def test_geometry_mismatch_is_reported(oracle):
    """A container decoded with another geometry than it was written with is
    refused (the header names its own), not turned into garbage."""
    from neuzip_amd import _lib

    n = 200_000
    bits = bf16_bits_normal(n, 8)
    comp, packed = gpu_encode(bits, 7, 65536, 344)
    for chunk, lane in ((65536, 512), (131072, 256)):
        print(f"case mismatch chunk={chunk} lane={lane}", flush=True)
        pk = torch.cat([packed, torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")])  # sizes differ per geometry
        rc, _ = gpu_decode(comp, pk, n, 7, chunk, lane)
        assert rc == _lib.ERR_CORRUPT
    rc, out = gpu_decode(comp, packed, n, 7, 65536, 344)
    assert rc == 0 and np.array_equal(out, bits)


def test_ratio_close_to_entropy(oracle):
    n = 4096 * 4096
    bits = bf16_bits_normal(n, seed=0)
    exps = ((bits >> 7) & 0xFF).astype(np.uint8)
    bound = chunk_entropy_bytes(exps)
    comp, packed = gpu_encode(bits, 7)
    # bytes stored beyond the raw sign|mantissa bits (the packed stream gives
    # back 128 bytes per full segment to the coder's start states)
    effective = comp.numel() + packed.numel() - n
    overhead = effective / bound - 1.0
    print(f"container {comp.numel()} B, packed {packed.numel()} B, entropy bound {bound:.0f} B, "
          f"overhead {100 * overhead:.3f}%", flush=True)
    assert overhead < 0.01


def test_split_api(oracle):
    L, m = _lib()
    for n in (0, 5, 2048, 100_001):
        bits = bf16_bits_normal(n, seed=n)
        d = _to_dev(bits) if n else torch.empty(0, dtype=torch.int16, device="cuda")
        e = torch.zeros(max(n, 8), dtype=torch.uint8, device="cuda")
        f = torch.zeros(max(n, 8), dtype=torch.uint8, device="cuda")
        rc = L.nz_split(d.data_ptr(), n, e.data_ptr(), f.data_ptr(), 0, None, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, m.last_error()
        torch.cuda.synchronize()
        oe, of = oracle.split(bits, 7)
        assert np.array_equal(e[:n].cpu().numpy(), oe)
        assert np.array_equal(f[:n].cpu().numpy(), of)


def test_decode_output_policy_flags(oracle):
    """nz_decode writes the same values whether the output is written with
    ordinary or with streaming stores; asking for both is an argument error."""
    L, m = _lib()
    for s in (7, 1):
        bits = stress_bits(64, 4099, seed=40 + s)
        comp, packed = gpu_encode(bits, s)
        want = oracle.reconstruct(bits, s)
        for flags in (0, m.DECODE_STREAM_OUT, m.DECODE_RESIDENT_OUT, m.DECODE_CHECK | m.DECODE_STREAM_OUT):
            out = torch.zeros(bits.size, dtype=torch.int16, device="cuda")
            status = torch.zeros(2, dtype=torch.int32, device="cuda")
            rc = L.nz_decode(comp.data_ptr(), comp.numel(), packed.data_ptr(), bits.size, s, 131072, 256,
                             out.data_ptr(), status.data_ptr(), flags, 0, None, torch.cuda.current_stream().cuda_stream)
            assert rc == 0, m.last_error()
            torch.cuda.synchronize()
            assert int(status[0]) == 0
            assert np.array_equal(out.cpu().numpy().view(np.uint16), want)
        rc = L.nz_decode(comp.data_ptr(), comp.numel(), packed.data_ptr(), bits.size, s, 131072, 256,
                         out.data_ptr(), status.data_ptr(), m.DECODE_STREAM_OUT | m.DECODE_RESIDENT_OUT, 0, None,
                         torch.cuda.current_stream().cuda_stream)
        assert rc == m.ERR_ARG and "exclude" in m.last_error()


@pytest.mark.parametrize("lane,chunk", [(256, 131072), (128, 65536), (64, 32768)])
def test_segment_that_outgrows_its_word_staging(oracle, lane, chunk):
    """The encode kernel keeps a segment's words in LDS when the chunk's histogram
    says they fit.  A chunk whose exponents are constant except for one segment of
    uniformly random ones has a small estimate and one segment that emits several
    times the staging room: that chunk is coded a second time, through scratch
    memory, and the bytes are the oracle's all the same (as are those of its
    ordinary neighbours)."""
    rng = np.random.default_rng(lane)
    n = 5 * chunk + 999
    seg = 64 * lane
    bits = bf16_bits_normal(n, seed=lane + 1)
    odd = slice(2 * chunk, 3 * chunk)                    # chunk 2: exponent 120 everywhere ...
    b = bits[odd]
    b = (b & 0x807F) | (120 << 7)
    hot = slice(3 * seg, 4 * seg)                        # ... but in its fourth segment any exponent
    b[hot] = (b[hot] & 0x807F) | (rng.integers(0, 255, seg).astype(np.uint16) << 7)
    bits[odd] = b
    print(f"case lane={lane} chunk={chunk}", flush=True)
    comp, packed = gpu_encode(bits, 7, chunk, lane)
    o_comp, o_packed = oracle.compress_bf16(bits, 7, chunk, lane)
    assert np.array_equal(packed.cpu().numpy(), o_packed)
    assert np.array_equal(comp.cpu().numpy(), o_comp)
    rc, out = gpu_decode(comp, packed, n, 7, chunk, lane)
    assert rc == 0 and np.array_equal(out, bits)


def test_encode_replayed_from_a_graph(oracle):
    """nz_encode captured into a HIP graph and replayed on new contents of the same
    buffers: every replay runs the very same call (same arguments, same scratch),
    so the size announcements of the replay before carry this call's mark; the
    run count kept in the scratch tells them apart.  Every replay's bytes are the
    oracle's."""
    L, m = _lib()
    n, s, chunk, lane = 9 * 131072 + 4321, 7, 131072, 256
    d_in = torch.zeros(n, dtype=torch.int16, device="cuda")
    cap = L.nz_exp_bound_bytes(n, chunk, lane)
    ws_bytes = L.nz_encode_workspace_bytes(n, chunk, lane)
    comp = torch.zeros(cap, dtype=torch.uint8, device="cuda")
    stored = L.nz_packed_stored_bytes(n, s, chunk, lane)
    packed = torch.zeros(stored, dtype=torch.uint8, device="cuda")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    aux = torch.zeros(4, dtype=torch.int64, device="cuda")

    def encode():
        rc = L.nz_encode(d_in.data_ptr(), n, s, chunk, lane, packed.data_ptr(), comp.data_ptr(), cap,
                         ws.data_ptr(), ws_bytes, aux.data_ptr(), aux.data_ptr() + 8, None, 0, None,
                         torch.cuda.current_stream().cuda_stream)
        assert rc == 0, m.last_error()

    encode()                                     # outside the capture first (one-time set-up of the kernels)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        encode()
    for rep in range(4):
        # different data every time, sizes of the chunks included (the exponent spread changes)
        bits = bf16_bits_normal(n, seed=100 + rep) if rep % 2 == 0 else stress_bits(n // 1024 + 1, 1024, seed=rep)[:n]
        d_in.copy_(_to_dev(bits))
        print(f"case graph replay {rep}", flush=True)
        g.replay()
        torch.cuda.synchronize()
        assert int(aux[1].item()) & 0xFFFFFFFF == 0
        total = int(aux[0].item())
        o_comp, o_packed = oracle.compress_bf16(bits, s, chunk, lane)
        assert total == o_comp.size
        assert np.array_equal(comp[:total].cpu().numpy(), o_comp)
        assert np.array_equal(packed.cpu().numpy(), o_packed)


@pytest.mark.parametrize("chunk,lane,n", [(8192, 16, 12_000_017), (65536, 256, 80_000_000), (32768, 64, 60_000_001)])
def test_records_are_placed_across_many_windows_of_chunks(oracle, chunk, lane, n):
    """More chunks than a workgroup has threads (1465, 1221 and 1832 of them, workgroups
    of 512 and 256 threads): a chunk finds the records before it from the running
    total of an earlier chunk plus the sizes of the chunks after that one, over
    several windows if need be; the container is the oracle's, twice in a row
    (the second run meets the first run's announcements in the same scratch)."""
    bits = bf16_bits_normal(n, seed=chunk % 89)
    o_comp, o_packed = oracle.compress_bf16(bits, 7, chunk, lane, threads=8)
    for rep in range(2):
        print(f"case chunk={chunk} lane={lane} n={n} run {rep}", flush=True)
        comp, packed = gpu_encode(bits, 7, chunk, lane)
        assert np.array_equal(comp.cpu().numpy(), o_comp)
        assert np.array_equal(packed.cpu().numpy(), o_packed)
