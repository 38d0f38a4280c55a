"""The library's calls recorded into a HIP graph: every replay must give what the same calls give launched one by one.

The entry points only enqueue kernels on the stream they are given (no allocation, no synchronisation, no memset
nodes), so a caller may record a whole layer into one graph.  The graph is replayed several times with the program's
own eager work and synchronisations in between, and every replay is compared bit for bit with the eager results (the
kernels are deterministic: no atomics)."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32) * scale


@pytest.mark.parametrize("D,Hq,Hkv,S", [(64, 8, 8, 640), (128, 8, 2, 1100)])
def test_layer_sized_call_sequence_replays_like_eager_launches(device, D, Hq, Hkv, S):
    from picotron_amd import _lib, ops
    from picotron_amd.model import get_cos_sin
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    B, hidden, inter, vocab = 2, 512, 1024, 3000
    rows = B * S
    scale = 1 / math.sqrt(D)
    bf = torch.bfloat16
    q = rnd(B, Hq, S, D, seed=1).to(bf).to(device)
    k = rnd(B, Hkv, S, D, seed=2).to(bf).to(device)
    v = rnd(B, Hkv, S, D, seed=3).to(bf).to(device)
    do = rnd(B, Hq, S, D, seed=4).to(bf).to(device)
    cos, sin = get_cos_sin(S, D)
    cos, sin = cos.to(device), sin.to(device)
    x = rnd(rows, hidden, seed=5).to(bf).to(device)
    res = rnd(rows, hidden, seed=6).to(bf).to(device)
    w = (1 + 0.1 * rnd(hidden, seed=7)).to(bf).to(device)
    dy = rnd(rows, hidden, seed=8).to(bf).to(device)
    gate_up = rnd(rows, 2 * inter, seed=9).to(bf).to(device)
    dh = rnd(rows, inter, seed=10).to(bf).to(device)
    logits = rnd(rows, vocab, seed=11, scale=3.0).to(bf).to(device)
    targets = torch.randint(0, vocab, (rows,), generator=torch.Generator().manual_seed(12)).to(device)
    targets[::7] = -100
    ce_scale = torch.full((1,), 1.0 / rows, dtype=torch.float32, device=device)
    dq = torch.empty(B, Hq, S, D, dtype=bf, device=device)
    dk = torch.empty(B, Hkv, S, D, dtype=bf, device=device)
    dv = torch.empty_like(dk)

    def work():
        r = {}
        # attention with RoPE inside the kernels (k rotated by its own launch), forward and backward
        k_rot = ops.rope(k, cos, sin)
        out, lse, q_rot = ops.attn_fwd_rope(q, k_rot, v, cos, sin, scale, True)
        ops.attn_bwd_rope(do, q_rot, k_rot, v, out, lse, cos, sin, scale, True, dq, dk, dv)
        r.update(out=out, lse=lse, dq=dq, dk=dk, dv=dv)
        # the plain entry points too: separate delta pre-pass, fp32 gradients
        o2, l2 = ops.attn_fwd(q, k, v, scale, True)
        delta = ops.attn_bwd_preprocess(do, o2)
        g2 = ops.attn_bwd(do, q, k, v, l2, delta, scale, True, 0)
        r.update(o2=o2, l2=l2, dq2=g2[0], dk2=g2[1], dv2=g2[2])
        # residual + RMSNorm both ways
        y, rstd, res_out = ops.rmsnorm_fwd(x, w, 1e-5, False, residual=res, want_residual_out=True)
        dx, dw = ops.rmsnorm_bwd(dy, res_out, w, rstd, dresidual=dy, dw_dtype=bf)
        r.update(y=y, rstd=rstd, res_out=res_out, dx=dx, dw=dw)
        # the entry point that allocates nothing (its first call on a device, which looks up the address of its static
        # array, was made by the eager run above: that call must lie outside a capture)
        dx_s, dw_s = torch.empty_like(dx), torch.empty_like(dw)
        _lib.check(_lib.lib().pico_rmsnorm_bwd_static(
            P(dy), P(res_out), P(w), P(rstd), P(dy), P(dx_s), P(dw_s), _lib.PICO_BF16, rows, hidden, _lib.PICO_BF16,
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        r.update(dx_s=dx_s, dw_s=dw_s)
        # SwiGLU on the halves of one projection output
        gate, up = gate_up[:, :inter], gate_up[:, inter:]
        hmid = ops.swiglu_fwd(gate, up)
        dgate, dup = ops.swiglu_bwd(dh, gate, up)
        r.update(hmid=hmid, dgate=dgate, dup=dup)
        # cross-entropy
        loss, clse = ops.cross_entropy_fwd(logits, targets)
        dlogits = ops.cross_entropy_bwd(logits, targets, clse, ce_scale)
        r.update(loss=loss, clse=clse, dlogits=dlogits)
        return r

    eager = {name: t.clone() for name, t in work().items()}
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = work()
    other = rnd(256, 256, seed=13).to(device)
    for replay in range(4):
        for t in recorded.values():          # nothing of an earlier replay may survive
            t.fill_(float("nan"))
        other = other @ other.t() * 1e-3      # the program's own eager work between two replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, t in recorded.items():
            assert torch.equal(t, eager[name]), f"replay {replay}: {name} differs from the eager result"


def test_calls_from_several_host_threads_on_their_own_streams(device):
    """The library keeps no mutable state between calls (its last-error text is per thread, its once-only set-up
    is atomic): four host threads, each with a stream of its own, run the forward and backward repeatedly and get the
    results of a single-threaded run bit for bit (autograd calls backward from a thread of its own)."""
    import threading
    from picotron_amd import ops
    B, H, S, D = 2, 8, 384, 64
    scale = 1 / math.sqrt(D)
    bf = torch.bfloat16
    cases = []
    for t in range(4):
        q, k, v, do = (rnd(B, H, S, D, seed=20 + 4 * t + i).to(bf).to(device) for i in range(4))
        out, lse = ops.attn_fwd(q, k, v, scale, True)
        grads = ops.attn_bwd(do, q, k, v, lse, None, scale, True, 0, dq_dtype=bf, dkv_dtype=bf, out=out)
        cases.append((q, k, v, do, out, lse, grads))
    torch.cuda.synchronize()
    errors = []

    def worker(t):
        try:
            q, k, v, do, out0, lse0, grads0 = cases[t]
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(20):
                    out, lse = ops.attn_fwd(q, k, v, scale, True)
                    grads = ops.attn_bwd(do, q, k, v, lse, None, scale, True, 0, dq_dtype=bf, dkv_dtype=bf, out=out)
                stream.synchronize()
            ok = torch.equal(out, out0) and torch.equal(lse, lse0) and all(torch.equal(a, b) for a, b in zip(grads, grads0))
            if not ok:
                errors.append(f"thread {t}: results differ from the single-threaded run")
        except Exception as e:  # noqa: BLE001 -- reported by the main thread
            errors.append(f"thread {t}: {e!r}")

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
