"""Random-init decoder models of the shapes BASELINE.json names, for bench.py.

Only shapes and layer types matter here (all weights are N(0, 0.02) from a
seed, all inputs uniform random token ids): the benchmark measures the codec
inside a realistic sequence of Linear layers, not model quality.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def _init_linear(lin: torch.nn.Linear):
    lin.weight.data.normal_(0.0, 0.02)
    if lin.bias is not None:
        lin.bias.data.zero_()


class RMSNorm(torch.nn.Module):
    def __init__(self, d, eps=1e-5):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.ones(d))
        self.eps = eps

    def forward(self, x):
        v = x.float()
        v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + self.eps)
        return (v * self.weight.float()).to(x.dtype)


def _rope(x, pos, theta=500000.0):
    # x: [B, H, T, D]; pos: [T]
    d = x.shape[-1]
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, device=x.device, dtype=torch.float32) / d))
    ang = pos.float()[:, None] * inv[None, :]
    cos, sin = ang.cos()[None, None], ang.sin()[None, None]
    x1, x2 = x.float()[..., 0::2], x.float()[..., 1::2]
    out = torch.stack((x1 * cos - x2 * sin, x1 * sin + x2 * cos), dim=-1).flatten(-2)
    return out.to(x.dtype)


class LlamaBlock(torch.nn.Module):
    def __init__(self, d, n_q, n_kv, ffn):
        super().__init__()
        self.n_q, self.n_kv, self.hd = n_q, n_kv, d // n_q
        self.input_norm = RMSNorm(d)
        self.q_proj = torch.nn.Linear(d, n_q * self.hd, bias=False)
        self.k_proj = torch.nn.Linear(d, n_kv * self.hd, bias=False)
        self.v_proj = torch.nn.Linear(d, n_kv * self.hd, bias=False)
        self.o_proj = torch.nn.Linear(n_q * self.hd, d, bias=False)
        self.post_norm = RMSNorm(d)
        self.gate_proj = torch.nn.Linear(d, ffn, bias=False)
        self.up_proj = torch.nn.Linear(d, ffn, bias=False)
        self.down_proj = torch.nn.Linear(ffn, d, bias=False)
        for m in (self.q_proj, self.k_proj, self.v_proj, self.o_proj, self.gate_proj, self.up_proj, self.down_proj):
            _init_linear(m)

    def forward(self, x, pos, cache):
        B, T, _ = x.shape
        h = self.input_norm(x)
        q = self.q_proj(h).view(B, T, self.n_q, self.hd).transpose(1, 2)
        k = self.k_proj(h).view(B, T, self.n_kv, self.hd).transpose(1, 2)
        v = self.v_proj(h).view(B, T, self.n_kv, self.hd).transpose(1, 2)
        q, k = _rope(q, pos), _rope(k, pos)
        if cache is not None:
            if cache[0] is not None:
                k = torch.cat((cache[0], k), dim=2)
                v = torch.cat((cache[1], v), dim=2)
            cache[0], cache[1] = k, v
        rep = self.n_q // self.n_kv
        kk = k.repeat_interleave(rep, dim=1)
        vv = v.repeat_interleave(rep, dim=1)
        a = F.scaled_dot_product_attention(q, kk, vv, is_causal=(T > 1))
        x = x + self.o_proj(a.transpose(1, 2).reshape(B, T, -1))
        h = self.post_norm(x)
        return x + self.down_proj(F.silu(self.gate_proj(h)) * self.up_proj(h))


def _block_static(blk, x, posv, kc, vc, mask):
    """One decode step of a LlamaBlock against a preallocated cache: the new key
    and value go to row `posv` of kc / vc ([1, n_kv, Tmax, hd]); `mask` hides the
    rows not written yet.  Shapes never change, so the step can be captured."""
    B, T, _ = x.shape
    h = blk.input_norm(x)
    q = blk.q_proj(h).view(B, T, blk.n_q, blk.hd).transpose(1, 2)
    k = blk.k_proj(h).view(B, T, blk.n_kv, blk.hd).transpose(1, 2)
    v = blk.v_proj(h).view(B, T, blk.n_kv, blk.hd).transpose(1, 2)
    q, k = _rope(q, posv), _rope(k, posv)
    kc.index_copy_(2, posv, k)
    vc.index_copy_(2, posv, v)
    rep = blk.n_q // blk.n_kv
    kk = kc.repeat_interleave(rep, dim=1)
    vv = vc.repeat_interleave(rep, dim=1)
    a = F.scaled_dot_product_attention(q, kk, vv, attn_mask=mask)
    x = x + blk.o_proj(a.transpose(1, 2).reshape(B, T, -1))
    h = blk.post_norm(x)
    return x + blk.down_proj(F.silu(blk.gate_proj(h)) * blk.up_proj(h))


class LlamaShaped(torch.nn.Module):
    """32 layers, d=4096, 32 q / 8 kv heads, FFN 14336, vocab 128256 by default."""

    def __init__(self, layers=32, d=4096, n_q=32, n_kv=8, ffn=14336, vocab=128256):
        super().__init__()
        self.embed = torch.nn.Embedding(vocab, d)
        self.embed.weight.data.normal_(0.0, 0.02)
        self.layers = torch.nn.ModuleList([LlamaBlock(d, n_q, n_kv, ffn) for _ in range(layers)])
        self.norm = RMSNorm(d)
        self.lm_head = torch.nn.Linear(d, vocab, bias=False)  # left dense by convert()
        _init_linear(self.lm_head)

    def forward(self, ids, start, caches):
        pos = torch.arange(start, start + ids.shape[1], device=ids.device)
        x = self.embed(ids)
        for blk, c in zip(self.layers, caches):
            x = blk(x, pos, c)
        return self.lm_head(self.norm(x[:, -1:]))

    @torch.no_grad()
    def static_caches(self, t_max):
        dev = self.embed.weight.device
        blk = self.layers[0]
        mk = lambda: torch.zeros(1, blk.n_kv, t_max, blk.hd, dtype=self.embed.weight.dtype, device=dev)
        return [mk() for _ in self.layers], [mk() for _ in self.layers]

    @torch.no_grad()
    def prefill_static(self, prompt, kcs, vcs):
        """Eager prefill; leaves keys and values in the static caches; returns the logits of the last position."""
        caches = [[None, None] for _ in self.layers]
        logits = self.forward(prompt, 0, caches)
        T = prompt.shape[1]
        for (k, v), kc, vc in zip(caches, kcs, vcs):
            kc[:, :, :T].copy_(k)
            vc[:, :, :T].copy_(v)
        return logits

    @torch.no_grad()
    def step_static(self, tok, pos, kcs, vcs):
        """One token: `tok` [1, 1] int64, `pos` a 1-element int64 device tensor."""
        t_max = kcs[0].shape[2]
        mask = (torch.arange(t_max, device=tok.device) <= pos).view(1, 1, 1, t_max)
        x = self.embed(tok)
        for blk, kc, vc in zip(self.layers, kcs, vcs):
            x = _block_static(blk, x, pos, kc, vc, mask)
        return self.lm_head(self.norm(x))

    @torch.no_grad()
    def generate(self, prompt, steps):
        """Greedy decode: prefill the prompt, then `steps` single-token steps."""
        caches = [[None, None] for _ in self.layers]
        logits = self.forward(prompt, 0, caches)
        tok = logits.argmax(-1)
        out = [tok]
        t = prompt.shape[1]
        for _ in range(steps - 1):
            logits = self.forward(tok, t, caches)
            tok = logits.argmax(-1)
            out.append(tok)
            t += 1
        return torch.cat(out, dim=1)


class GPT2Block(torch.nn.Module):
    def __init__(self, d, heads):
        super().__init__()
        self.heads = heads
        self.ln1 = torch.nn.LayerNorm(d)
        self.qkv = torch.nn.Linear(d, 3 * d)
        self.proj = torch.nn.Linear(d, d)
        self.ln2 = torch.nn.LayerNorm(d)
        self.fc = torch.nn.Linear(d, 4 * d)
        self.fc2 = torch.nn.Linear(4 * d, d)
        for m in (self.qkv, self.proj, self.fc, self.fc2):
            _init_linear(m)

    def forward(self, x):
        B, T, D = x.shape
        q, k, v = self.qkv(self.ln1(x)).view(B, T, 3, self.heads, D // self.heads).permute(2, 0, 3, 1, 4)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        x = x + self.proj(a.transpose(1, 2).reshape(B, T, D))
        return x + self.fc2(F.gelu(self.fc(self.ln2(x))))


class GPT2Shaped(torch.nn.Module):
    """24 layers, d=1024, 16 heads, vocab 50257 by default (GPT-2 medium shape)."""

    def __init__(self, layers=24, d=1024, heads=16, vocab=50257, ctx=1024):
        super().__init__()
        self.wte = torch.nn.Embedding(vocab, d)
        self.wpe = torch.nn.Embedding(ctx, d)
        self.wte.weight.data.normal_(0.0, 0.02)
        self.wpe.weight.data.normal_(0.0, 0.02)
        self.blocks = torch.nn.ModuleList([GPT2Block(d, heads) for _ in range(layers)])
        self.ln_f = torch.nn.LayerNorm(d)
        self.lm_head = torch.nn.Linear(d, vocab, bias=False)
        _init_linear(self.lm_head)

    def forward(self, ids):
        T = ids.shape[1]
        x = self.wte(ids) + self.wpe(torch.arange(T, device=ids.device))[None]
        for b in self.blocks:
            x = b(x)
        return self.lm_head(self.ln_f(x))


class CompressedAdamW:
    """AdamW for compressed parameters: decompress, update, re-compress under the
    same handle (the read -> update -> write idiom of neuzip/__init__.py:25-35).
    The update itself is torch's own multi-tensor AdamW on the decoded weights,
    with moments in the weights' dtype as ``torch.optim.AdamW`` keeps them, so a
    lossless manager trains exactly like the dense model."""

    def __init__(self, params, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, group=1):
        """``group``: parameters are read, updated and written back ``group`` at a
        time (the Linears of one block), so that a per-block decode serves all
        of them before the first write makes it stale."""
        self.params = list(params)
        self.group = max(1, int(group))
        self.lr, self.b1, self.b2, self.eps, self.wd = lr, betas[0], betas[1], eps, weight_decay
        self.state = {}

    @torch.no_grad()
    def step(self):
        from torch.optim.adamw import adamw

        todo = [p for p in self.params if p._gradient is not None]
        for at in range(0, len(todo), self.group):
            batch = todo[at:at + self.group]
            weights, grads, m1, m2, steps = [], [], [], [], []
            for p in batch:
                w = p.shared()  # decompress; updated in place, then written back under the same handle
                st = self.state.get(p._handle)
                if st is None:
                    st = (torch.zeros_like(w), torch.zeros_like(w), torch.tensor(0.0, dtype=torch.float32))
                    self.state[p._handle] = st
                weights.append(w)
                grads.append(p._gradient.to(w.dtype).view_as(w))
                m1.append(st[0])
                m2.append(st[1])
                steps.append(st[2])
            adamw(weights, grads, m1, m2, [], steps, foreach=True, amsgrad=False, beta1=self.b1, beta2=self.b2,
                  lr=self.lr, weight_decay=self.wd, eps=self.eps, maximize=False)
            if len(batch) > 1:
                batch[0]._manager.write_many(weights, [p._handle for p in batch])  # re-compress, one sync
            else:
                batch[0]._manager.write(weights[0], batch[0]._handle)
            for p in batch:
                p._gradient = None
                p.grad = None


class ReferenceLoopSGD:
    """The update the reference's training example applies to compressed
    parameters, statement for statement (examples/training/train_clm.py:822-833):
    ``write(read(handle).add_(gradient, alpha=-lr), handle)``, one parameter
    after the other."""

    def __init__(self, params, lr=1e-4):
        self.params = list(params)
        self.lr = lr

    @torch.no_grad()
    def step(self):
        for p in self.params:
            if getattr(p, "_gradient", None) is not None:
                p._manager.write(p._manager.read(p._handle).add_(p._gradient, alpha=-self.lr), p._handle)
                p._gradient = None
                p.grad = None


def paired_parameters(dense: torch.nn.Module, comp: torch.nn.Module):
    """``[(name, dense parameter, its counterpart in the converted twin)]``: for a
    compressed Linear the counterpart of ``weight`` is the ``neuzip_amd.nn.Parameter``."""
    from neuzip_amd.nn import Linear as CompressedLinearModule

    dense_mods = dict(dense.named_modules())
    pairs = []
    for name, mod in comp.named_modules():
        twin = dense_mods[name]
        if isinstance(mod, CompressedLinearModule):
            pairs.append((f"{name}.weight", twin.weight, mod._p))
            if mod.bias is not None:
                pairs.append((f"{name}.bias", twin.bias, mod.bias))
            continue
        for pname, p in mod.named_parameters(recurse=False):
            pairs.append((f"{name}.{pname}" if name else pname, getattr(twin, pname), p))
    return pairs


def _same_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    a, b = a.detach().reshape(-1), b.detach().reshape(-1)
    if a.dtype == torch.bfloat16:
        return bool(torch.equal(a.view(torch.int16), b.view(torch.int16)))
    return bool(torch.equal(a, b))


def lockstep_adamw(dense, comp, manager, ids_for_step, steps, group, lr=1e-4, probe_dense_twice=True):
    """Train ``dense`` (torch.optim.AdamW) and ``comp`` (the same model converted
    by ``manager``: CompressedAdamW re-compressing with ``write_many``) side by
    side on the same token ids, and separate what the codec is responsible for
    from what the GEMM / attention kernels are responsible for.

    Per step both models run forward and backward; losses and gradients are
    compared and the first tensor whose gradient differs is recorded (the
    weights going in are identical, so such a difference belongs to the
    forward / backward kernels, never to the codec).  Then the DENSE gradients
    are handed to both optimizers, both step, and every weight of the
    compressed model (decoded from its store) must equal the dense model's
    weight bit for bit: that is the part the codec and the compressed
    optimizer answer for.  With ``probe_dense_twice`` the dense model's
    backward is run twice per step on the same input: if its own gradients
    differ between the two runs, the kernels are not run-to-run deterministic
    and no loss curve can be expected to repeat.

    -> dict of findings; ``first_weight_mismatch`` must be None."""
    import neuzip_amd

    pairs = paired_parameters(dense, comp)
    packed = [(n, d, c) for n, d, c in pairs if isinstance(c, neuzip_amd.nn.Parameter)]
    plain = [(n, d, c) for n, d, c in pairs if not isinstance(c, neuzip_amd.nn.Parameter)]
    opt_dense = torch.optim.AdamW([d for _, d, _ in pairs], lr=lr)
    opt_packed = CompressedAdamW([c for _, _, c in packed], lr=lr, group=group)
    opt_plain = torch.optim.AdamW([c for _, _, c in plain], lr=lr)

    def loss_of(model, ids):
        logits = model(ids[:, :-1])
        return F.cross_entropy(logits.float().reshape(-1, logits.shape[-1]), ids[:, 1:].reshape(-1))

    def grad_of(c):
        return c._gradient if isinstance(c, neuzip_amd.nn.Parameter) else c.grad

    out = {"steps": steps, "losses_equal": 0, "gradients_equal": 0, "first_loss_mismatch": None,
           "first_gradient_mismatch": None, "first_weight_mismatch": None, "dense_repeats_itself": None,
           "max_loss_gap": 0.0}
    repeats = 0
    for step in range(steps):
        ids = ids_for_step(step)
        if probe_dense_twice:
            loss_of(dense, ids).backward()
            first = [d.grad.clone() for _, d, _ in pairs]
            opt_dense.zero_grad(set_to_none=True)
        loss_d = loss_of(dense, ids)
        loss_d.backward()
        if probe_dense_twice:
            repeats += all(_same_bits(g, d.grad) for g, (_, d, _) in zip(first, pairs))
            del first
        loss_c = loss_of(comp, ids)
        loss_c.backward()
        same_loss = bool(torch.equal(loss_d.detach(), loss_c.detach()))
        out["losses_equal"] += same_loss
        out["max_loss_gap"] = max(out["max_loss_gap"], abs(float(loss_d.detach()) - float(loss_c.detach())))
        if not same_loss and out["first_loss_mismatch"] is None:
            out["first_loss_mismatch"] = step
        differing = [n for n, d, c in pairs if not _same_bits(d.grad, grad_of(c).view_as(d.grad))]
        out["gradients_equal"] += not differing
        if differing and out["first_gradient_mismatch"] is None:
            out["first_gradient_mismatch"] = {"step": step, "tensor": differing[0], "tensors": len(differing)}
        # the same numbers into both optimizers
        with torch.no_grad():
            for _, d, c in packed:
                c._gradient = d.grad.clone()
            for _, d, c in plain:
                c.grad = d.grad.clone()
        opt_dense.step()
        opt_packed.step()
        opt_plain.step()
        opt_dense.zero_grad(set_to_none=True)
        opt_plain.zero_grad(set_to_none=True)
        with torch.no_grad():
            for n, d, c in pairs:
                w = manager.read(c._handle) if isinstance(c, neuzip_amd.nn.Parameter) else c.data
                if not _same_bits(d.data, w.view_as(d.data)):
                    out["first_weight_mismatch"] = {"step": step, "tensor": n}
                    return out
    if probe_dense_twice:
        out["dense_repeats_itself"] = f"{repeats} of {steps}"
    return out
