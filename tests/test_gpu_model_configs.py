"""The two model-shaped BASELINE workloads at full width and reduced depth:

* a Llama-3-8B-shaped decoder (d=4096, 32 q / 8 kv heads, FFN 14336, vocab
  128256; two layers here, 512-token prompt, 16 single-token steps) converted
  the way the reference's user does it (``import neuzip;
  neuzip.Manager(precision=7).convert(model)``): stored weights against the
  oracle and inside the size budget, logits of every decompress-then-GEMM mode
  (per Linear, per block, decode-ahead, HIP-graph replays) bit-equal to the
  dense model's, the fused matrix-vector product (what the unchanged caller's
  single-token steps run) within its floating-point tolerance and bit-equal to
  nz_manager_gemv_batch called by hand;
* a GPT-2-medium-shaped model (d=1024, 16 heads, vocab 50257; two layers here)
  trained with AdamW for 20 steps, batch 8 x 1024, weights re-compressed after every step
  (the read -> update -> write idiom of neuzip/__init__.py:25-35 and
  examples/training/train_clm.py:822-833): fed the dense run's gradients, every
  decoded weight equals the dense AdamW weight bit for bit after every step.
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _bits(t):
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1)


def _entropy_bytes(exps: np.ndarray) -> float:
    from conftest import chunk_entropy_bytes

    return chunk_entropy_bytes(exps)


def _llama(layers, seed):
    from bench_models import LlamaShaped

    torch.manual_seed(seed)
    with torch.device("cuda"):
        torch.set_default_dtype(torch.bfloat16)
        try:
            model = LlamaShaped(layers=layers)
        finally:
            torch.set_default_dtype(torch.float32)
    return model.eval()


def test_llama_shaped_decoder_all_modes(oracle):
    import neuzip
    import neuzip_amd

    model = _llama(layers=2, seed=11)
    names = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")
    shapes = {"q_proj": (4096, 4096), "k_proj": (1024, 4096), "v_proj": (1024, 4096), "o_proj": (4096, 4096),
              "gate_proj": (14336, 4096), "up_proj": (14336, 4096), "down_proj": (4096, 14336)}
    dense_w = {(li, n): getattr(blk, n).weight.data.clone() for li, blk in enumerate(model.layers) for n in names}
    assert all(tuple(dense_w[(0, n)].shape) == shapes[n] for n in names)

    T, steps = 512, 16
    g = torch.Generator(device="cuda").manual_seed(3)
    prompt = torch.randint(0, 128256, (1, T), device="cuda", generator=g)
    kcs, vcs = model.static_caches(T + steps + 2)
    tok_buf = torch.zeros(1, 1, dtype=torch.int64, device="cuda")
    pos_buf = torch.zeros(1, dtype=torch.int64, device="cuda")

    def run(graph=None):
        """prefill + `steps` greedy single-token steps -> list of logits (prefill first)"""
        with torch.no_grad():
            logits = model.prefill_static(prompt, kcs, vcs)
            outs = [logits.clone()]
            tok = logits.argmax(-1)
            for i in range(steps):
                pos_buf.fill_(T + i)
                tok_buf.copy_(tok.view(1, 1))
                if graph is None:
                    logits = model.step_static(tok_buf, pos_buf, kcs, vcs)
                else:
                    graph[0].replay()
                    logits = graph[1]
                outs.append(logits.clone())
                tok = logits.argmax(-1)
                float(logits.float().sum())  # eager work and a host synchronisation between replays
        return outs

    def capture(finish=None):
        with torch.no_grad():
            model.prefill_static(prompt, kcs, vcs)
            pos_buf.fill_(T)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(2):
                    model.step_static(tok_buf, pos_buf, kcs, vcs)
                if finish:
                    finish()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                logits = model.step_static(tok_buf, pos_buf, kcs, vcs)
                if finish:
                    finish()
        return gr, logits

    print("case llama dense", flush=True)
    want = run()

    mgr = neuzip.Manager(precision=7)  # the reference's call, no extension arguments
    mgr.convert(model)
    torch.cuda.empty_cache()
    # every stored weight, read back, is the oracle's reconstruction of the dense bits,
    # and what is stored for its exponents stays within 1.01 x their order-0 entropy
    for li, blk in enumerate(model.layers):
        for n in names:
            lin = getattr(blk, n)
            assert isinstance(lin, neuzip_amd.nn.Linear) and lin.weight.numel() == 0
            bits = _bits(dense_w[(li, n)])
            got = _bits(mgr.read(lin.weight._handle))
            assert np.array_equal(got, oracle.reconstruct(bits, 7)), (li, n)
            exps = ((bits >> 7) & 0xFF).astype(np.uint8)
            over = (mgr.size(lin.weight._handle) - bits.size) / _entropy_bytes(exps)
            assert over <= 1.01, (li, n, over, mgr._be.geometry(lin.weight._handle))
    assert isinstance(model.lm_head, torch.nn.Linear) and isinstance(model.embed, torch.nn.Embedding)
    del dense_w

    def same(got, tag):
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f"{tag}: logits differ at {'prefill' if i == 0 else f'step {i}'}"

    # the unchanged caller: prefill by decompress-then-GEMM (the dense model's logits,
    # bit for bit), single-token steps by the fused product
    print("case llama unchanged caller", flush=True)
    assert mgr.fused_rows
    plain = run()
    plain_graph = run(capture())
    assert torch.equal(plain[0], want[0])
    for a, b in zip(plain[1:2], want[1:2]):  # same token, same cache: only the summation order differs
        rel = float((a.float() - b.float()).norm() / b.float().norm())
        assert rel < 0.02, rel
    for a, b in zip(plain, plain_graph):
        assert torch.equal(a, b)
    # q/k/v and gate/up were recognised as runs that share their activation: one launch each
    runs = sorted(len(r[0]) for r in mgr._be._runs.values())
    assert runs == [2, 2, 3, 3], runs
    mgr.group_rows = False  # every Linear a launch of its own: the same numbers
    for a, b in zip(plain, run()):
        assert torch.equal(a, b)
    mgr.group_rows = True

    mgr.fused_rows = False  # every call by decompress-then-GEMM: the dense model's logits exactly
    print("case llama per_linear eager", flush=True)
    same(run(), "per_linear eager")
    print("case llama per_linear graph", flush=True)
    same(run(capture()), "per_linear graph")
    for ahead in (False, True):
        tag = "per_block_ahead" if ahead else "per_block"
        print(f"case llama {tag} eager", flush=True)
        with neuzip_amd.DecompressAhead(mgr, model, ahead=ahead):
            same(run(), tag + " eager")
        print(f"case llama {tag} graph", flush=True)
        da = neuzip_amd.DecompressAhead(mgr, model, ahead=ahead, wrap=False)
        with da:
            same(run(capture(finish=da.join)), tag + " graph")
        del da

    # fused decode + matrix-vector product: every matrix of a block at its stored
    # geometry against an fp64 product (bf16 output: half an ulp is 2^-9 relative,
    # fp32 partial sums add a little relative to the sum of magnitudes)
    print("case llama fused per matrix", flush=True)
    blk = model.layers[1]
    for n in names:
        lin = getattr(blk, n)
        x = torch.randn(lin.in_features, device="cuda", generator=g).to(torch.bfloat16)
        y = torch.zeros(lin.out_features, dtype=torch.bfloat16, device="cuda")
        mgr._be.gemv_batch((ctypes.c_char_p * 1)(lin.weight._handle.encode()), x, None, [y])
        w = lin.weight().double()
        ref = w @ x.double()
        tol = 2.0 ** -8 * ref.abs() + 1e-5 * (w.abs() @ x.double().abs()) + 2.0 ** -36
        assert bool(((y.double() - ref).abs() <= tol).all()), n
        del w
    # and through the model: fused single-token steps stay close to the dense
    # logits (its summation order is its own), graph replays equal the eager run
    print("case llama fused model", flush=True)
    mgr.fused_rows = True
    fused = neuzip_amd.FusedGemv(mgr, model)
    with fused:  # not traced yet: every Linear a launch of its own through nz_manager_gemv_batch ...
        by_hand = run()
    for a, b in zip(plain, by_hand):  # ... which is what the unchanged caller's steps ran
        assert torch.equal(a, b)
    with torch.no_grad():
        model.prefill_static(prompt, kcs, vcs)
        pos_buf.fill_(T)
        fused.trace(lambda: model.step_static(tok_buf, pos_buf, kcs, vcs))
    assert sorted(len(gr.handles) for gr in fused._groups) == [1, 1, 1, 1, 2, 2, 3, 3]  # q/k/v and gate/up share a launch
    with fused:
        eager = run()
        replay = run(capture())
    assert torch.equal(eager[0], want[0])  # the prefill keeps the decompress-then-GEMM path
    for a, b in zip(eager[1:2], want[1:2]):  # same token, same cache: only the summation order differs
        rel = float((a.float() - b.float()).norm() / b.float().norm())
        assert rel < 0.02, rel
    for a, b in zip(eager, replay):
        assert torch.equal(a, b)
    mgr._be.check()


def test_gpt2_shaped_adamw_recompress_matches_dense():
    import neuzip_amd
    from bench_models import GPT2Shaped, lockstep_adamw

    def build():
        torch.manual_seed(17)
        with torch.device("cuda"):
            torch.set_default_dtype(torch.bfloat16)
            try:
                return GPT2Shaped(layers=2, ctx=1024)
            finally:
                torch.set_default_dtype(torch.float32)

    import neuzip

    dense, comp = build(), build()
    mgr = neuzip.Manager(precision=7)  # the reference's call, no extension arguments
    mgr.convert(comp)
    packed = [p for p in comp.parameters() if isinstance(p, neuzip_amd.nn.Parameter)]
    assert len(packed) == 8 and sorted(tuple(p._shape) for p in packed)[-1] == (4096, 1024)
    steps = 20
    g = torch.Generator(device="cuda").manual_seed(5)
    batches = [torch.randint(0, 50257, (8, 1024), device="cuda", generator=g) for _ in range(steps)]
    print("case gpt2 lockstep", flush=True)
    with neuzip_amd.DecompressAhead(mgr, comp, ahead=False):
        found = lockstep_adamw(dense, comp, mgr, lambda i: batches[i], steps=steps, group=4)
    print("lockstep findings:", found, flush=True)
    # what the codec and the compressed optimizer answer for: identical weights after every step
    assert found["first_weight_mismatch"] is None, found
    # the weights going into every step are identical, so the two forward passes
    # compute the same function; their kernels may round differently
    assert found["max_loss_gap"] < 1e-2, found
    # after 20 updates every stored weight is still inside the size budget
    for p in packed:
        bits = _bits(p())
        exps = ((bits >> 7) & 0xFF).astype(np.uint8)
        over = (mgr.size(p._handle) - bits.size) / _entropy_bytes(exps)
        assert over <= 1.01, (tuple(p._shape), over, mgr._be.geometry(p._handle))
    mgr._be.check()


def test_manager_size_by_the_references_formula():
    """size(handle, reference_accounting=True) adds the ceil(N / 1024) bytes the
    reference counts for its unused normalizer buffer (cuda/high_level.cu:89-93,208-221)."""
    import neuzip_amd

    w = torch.randn(300, 1000, device="cuda").to(torch.bfloat16)
    mgr = neuzip_amd.Manager()
    h = mgr.write(w)
    assert mgr.size(h, reference_accounting=True) == mgr.size(h) + (300_000 + 1023) // 1024
    assert mgr.size("nope", reference_accounting=True) == 0
    mgn = neuzip_amd.Manager(precision=3, normalizer_size=64)
    h = mgn.write(w)
    assert mgn.size(h, reference_accounting=True) == mgn.size(h)  # normalizers on: already counted
