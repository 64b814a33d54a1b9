"""Manager calls against streams, graph capture and recycled input memory.

* a call that may allocate or wait on the host is refused while its stream is
  being captured, with an error and without invalidating the capture; reads
  and products that need neither are captured and replay exactly;
* calls that share the manager's scratch memory are ordered on the device when
  they arrive on different streams;
* an in-place rewrite may return while the encode still reads its input: the
  Python layer keeps a temporary's memory from being reused by another stream
  (``record_stream``), and memory recycled on the same stream is safe by stream
  order; both against the oracle's bytes;
* the size budget's setter."""
import ctypes

import numpy as np
import pytest

from conftest import bf16_bits_normal

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def from_bits(bits, shape):
    return torch.from_numpy(bits.view(np.int16).copy()).cuda().view(torch.bfloat16).view(shape)


def bits_of(t):
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1)


def test_blocking_calls_are_refused_under_capture_and_the_capture_survives():
    import neuzip_amd

    mgr = neuzip_amd.Manager(lane_symbols=256)
    n = 6 * 131072 + 99
    w = from_bits(bf16_bits_normal(n, seed=1), (n,))
    w2 = (w.float() * 1.01).to(torch.bfloat16)
    h = mgr.write(w)
    out = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    mgr._be.read_into(h, out)  # warm: nothing left to allocate for a read
    torch.cuda.synchronize()
    out.zero_()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        print("case write under capture", flush=True)
        with pytest.raises(ValueError, match="being captured"):
            mgr.write(w2, h)
        with pytest.raises(ValueError, match="being captured"):
            mgr.write(w2, "other")
        with pytest.raises(ValueError, match="being captured"):
            mgr.write_many([w2], [h])
        print("case read under capture", flush=True)
        mgr._be.read_into(h, out)  # settled entry: recorded
    # the refusals left the capture valid: the graph exists and replays the read
    for _ in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, w)
    # the refused writes changed nothing
    assert torch.equal(mgr.read(h), w) and mgr.size("other") == 0
    # a read of an entry whose in-place rewrite is still unsettled has to wait on the host: refused as well
    mgr.write(w2, h)  # in place (same size class): pending until settled
    g2 = torch.cuda.CUDAGraph()
    refused = False
    with torch.cuda.graph(g2):
        try:
            mgr._be.read_into(h, out)
        except ValueError as e:
            refused = "being captured" in str(e)
        out.add_(0)  # the capture holds something either way
    g2.replay()
    torch.cuda.synchronize()
    assert torch.equal(mgr.read(h), w2)
    if refused:
        print("pending read was refused under capture", flush=True)
    else:  # the rewrite had been settled already: the read was recorded
        assert torch.equal(out, w2)
    mgr._be.check()


def test_scratch_users_on_different_streams_are_ordered(oracle):
    """Two streams alternate writes of large tensors through ONE manager, with no
    host synchronisation and no event of the caller's between them: both use the
    manager's encode workspace, so the library has to order them."""
    import neuzip_amd

    mgr = neuzip_amd.Manager(lane_symbols=256)
    n = 48 * 131072 + 5
    ws = [from_bits(bf16_bits_normal(n, seed=40 + i), (n,)) for i in range(4)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    hs = []
    for rnd in range(3):  # first round sizes the entries, the next ones rewrite them in place
        for i, w in enumerate(ws):
            st = streams[i % 2]
            with torch.cuda.stream(st):
                print(f"case round {rnd} tensor {i} on stream {i % 2}", flush=True)
                if rnd == 0:
                    hs.append(mgr.write(w))
                else:
                    mgr.write(w, hs[i])
    torch.cuda.synchronize()
    for i, (w, h) in enumerate(zip(ws, hs)):
        o_comp, o_packed = oracle.compress_bf16(bits_of(w), 7, 131072, 256, threads=8)
        comp, packed, _ = mgr._be.export(h)
        assert np.array_equal(comp.numpy(), o_comp) and np.array_equal(packed.numpy(), o_packed), i
        assert torch.equal(mgr.read(h), w)
    mgr._be.check()


def test_rewrite_from_a_temporary_whose_memory_is_recycled(oracle):
    """write() of an in-place rewrite returns while the encode kernel may still be
    reading the dense input.  The input here is a temporary that is dropped the
    moment write() returns, and the caching allocator hands its memory to the
    next tensor, which is overwritten at once: on the same stream (ordered after
    the encode by the stream), and - for a temporary that was produced on a
    second stream - on that stream, which may only get the memory back once the
    encode is done, because write() recorded its use."""
    import neuzip_amd

    mgr = neuzip_amd.Manager(lane_symbols=256)
    n = 40 * 131072 + 1234
    base = from_bits(bf16_bits_normal(n, seed=9), (n,))
    h = mgr.write(base)
    mgr.read(h)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    for step in range(1, 7):
        scale = 1.0 + 0.002 * step
        want = (base.float() * scale).to(torch.bfloat16)
        o_comp, o_packed = oracle.compress_bf16(bits_of(want), 7, 131072, 256, threads=8)
        torch.cuda.synchronize()
        print(f"case step {step}", flush=True)
        if step % 2:
            tmp = (base.float() * scale).to(torch.bfloat16)  # a temporary with no other owner
            ptr = tmp.data_ptr()
            mgr.write(tmp, h)
            del tmp  # back to the allocator while the encode may still be running
            junk = torch.full((n,), 7.0, dtype=torch.bfloat16, device="cuda")  # same stream: may reuse the block
        else:
            with torch.cuda.stream(side):  # produced on another stream: the block belongs to that stream's pool
                tmp = (base.float() * scale).to(torch.bfloat16)
            torch.cuda.current_stream().wait_stream(side)
            ptr = tmp.data_ptr()
            mgr.write(tmp, h)  # encodes on the current stream
            del tmp
            with torch.cuda.stream(side):  # must not be handed the block before the encode is done
                junk = torch.full((n,), 7.0, dtype=torch.bfloat16, device="cuda")
        reused = junk.data_ptr() == ptr
        comp, packed, _ = mgr._be.export(h)
        assert np.array_equal(comp.numpy(), o_comp) and np.array_equal(packed.numpy(), o_packed), (step, reused)
        assert torch.equal(mgr.read(h), want)
        del junk
    batches, outgrown = mgr._be.rewrite_stats()
    assert batches >= 5 and outgrown == 0  # these were in-place rewrites
    mgr._be.check()


def test_size_budget_setter():
    import neuzip_amd
    from neuzip_amd import _lib

    L = _lib.load()
    mgr = neuzip_amd.Manager()
    assert mgr._be.size_budget == pytest.approx(_lib.DEFAULT_SIZE_BUDGET)
    for bad in (1.0, 1.002, 2.5, float("nan")):
        assert L.nz_manager_set_size_budget(mgr._be._h, ctypes.c_double(bad)) != 0
    assert mgr._be.size_budget == pytest.approx(_lib.DEFAULT_SIZE_BUDGET)
    n = 4096 * 1024
    w = from_bits(bf16_bits_normal(n, seed=2), (n,))
    h = mgr.write(w)
    assert mgr._be.geometry(h) == (135168, 264)
    assert mgr._be.in_budget(n, 135168, 264) and not mgr._be.in_budget(n, 131072, 256)
    assert 1.009 < mgr._be.estimated_size_ratio(n, 131072, 256) < 1.0101
    assert mgr._be.estimated_size_ratio(n, 131072, 100) == 0.0  # not a valid geometry
    loose = neuzip_amd.Manager(size_budget=1.02)
    h2 = loose.write(w)
    assert loose._be.geometry(h2) == (131072, 256) and loose._be.size_budget == pytest.approx(1.02)
    tight = neuzip_amd.Manager(size_budget=1.006)
    h3 = tight.write(w)
    chunk, lane = tight._be.geometry(h3)
    assert chunk == 512 * lane and lane > 400 and tight.size(h3) < mgr.size(h) < loose.size(h2)
    for m_, h_ in ((mgr, h), (loose, h2), (tight, h3)):
        assert torch.equal(m_.read(h_), w)
