"""Benchmark of the hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (BASELINE.json configs[1]): causal ring attention, q/k/v bf16 [B=4, H=32, S=1024, D=64],
cp_size = 4 (chunks of 256).  One "step" is forward + backward of the ring for ALL four cp ranks on the
one GPU: rank r attends its 256-query chunk over the K/V chunks 0..r (diagonal chunk masked, earlier
chunks dense) and its backward adds into dK/dV of those chunks.  The four ranks are batched into one
launch per direction: the grid's query-tile index enumerates (rank, tile of the rank's chunk), every
workgroup walks the chunks its rank would receive, the online softmax carries across them (no score
matrix, no per-chunk partial result and no separate merge pass touches HBM), and dK/dV of a chunk are
summed over the ranks inside the kernel.  Launches per step: forward, delta pre-pass, backward dK/dV,
backward dQ (gradients are written in bf16 directly).  The step is recorded once into a HIP graph and replayed K times; inputs are resident
in HBM before the timed region.

value = algorithmic FLOPs of the step (7 * B*H*S^2*D = 60.13 GFLOP: forward 4 and backward 10 FLOPs
per (query, key, d) triple, the masked diagonal chunk counted half) / measured time.

The JSON line also carries
  roofline      the dominant kernel (attention backward) against the dense bf16 MFMA peak,
  cpu_baseline  the CPU oracle (plain torch restatement of picotron's blockwise ring attention, fp32)
                timed on this host,
  extras        forward / backward split; the same step as one launch per rank and as one launch per
                ring step (the reference's schedule); the bandwidth kernels (RMSNorm, RoPE, SwiGLU)
                against the 8 TB/s HBM peak; a SmolLM-1.7B-shaped training step (tokens/s).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
HBM_PEAK_GBS = 8000.0
# HBM bytes of one dK/dV launch at the bench shape, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by a copy
# kernel of known size (see profiles/); None until measured
TRAFFIC_BYTES_DKDV = 107.8e6


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the extra kernels")
    ap.add_argument("--no-train", action="store_true", help="skip the SmolLM-1.7B- and Llama-2-7B-shaped training steps")
    ap.add_argument("--train-step", choices=["smollm_1p7b", "llama2_7b"], default=None,
                    help="run only that training step (for a kernel trace of it) and print its figures")
    ap.add_argument("--probe", nargs="?", const="configs1", default=None, choices=["configs1", "configs4", "ring_api"],
                    help="counter probe: a few launches of a plain copy of known size and of each attention kernel "
                         "at the bench shape (configs1) or at configs[4]'s shape (rank 7 of 8, head_dim 128), nothing else "
                         "(for rocprofv3 --pmc)")
    return ap.parse_args()


class RingBench:
    """State + one step of the all-ranks ring (fused launches) for configs[1]."""

    def __init__(self, torch, ops, B=4, H=32, S=1024, D=64, W=4, device="cuda"):
        self.torch, self.ops = torch, ops
        self.B, self.H, self.S, self.D, self.W = B, H, S, D, W
        self.Sc = S // W
        self.scale = 1.0 / math.sqrt(D)
        g = torch.Generator().manual_seed(0)
        q = torch.randn(B, H, S, D, generator=g) * self.scale   # "scaled by 1/sqrt(D) on q"
        k = torch.randn(B, H, S, D, generator=g)
        v = torch.randn(B, H, S, D, generator=g)
        do = torch.randn(B, H, S, D, generator=g)
        self.host = tuple(t.to(torch.bfloat16) for t in (q, k, v, do))
        self.q, self.k, self.v, self.do = (t.to(device) for t in self.host)
        f32 = dict(dtype=torch.float32, device=device)
        self.out = torch.empty(B, H, S, D, dtype=torch.bfloat16, device=device)
        self.lse = torch.empty(W, B, H, self.Sc, **f32)
        self.delta = torch.empty(W, B, H, self.Sc, **f32)
        self.dq_acc = torch.empty(W, B, H, self.Sc, D, **f32)
        self.dk_acc = torch.empty(B, H, S, D, **f32)
        self.dv_acc = torch.empty(B, H, S, D, **f32)
        self.lse_b = torch.empty(B, H, S, **f32)
        self.delta_b = torch.empty(B, H, S, **f32)
        self.dq_b = torch.empty(B, H, S, D, dtype=torch.bfloat16, device=device)
        self.dk_b = torch.empty(B, H, S, D, dtype=torch.bfloat16, device=device)
        self.dv_b = torch.empty(B, H, S, D, dtype=torch.bfloat16, device=device)

    def flops(self):
        blocks = self.W * (self.W + 1) / 2 - self.W / 2  # diagonal blocks count half
        per_block = self.B * self.H * self.Sc * self.Sc * self.D
        return 4 * per_block * blocks, 10 * per_block * blocks

    def _views(self, r):
        Sc = self.Sc
        sl_q = slice(r * Sc, (r + 1) * Sc)
        sl_k = slice(0, (r + 1) * Sc)
        return (self.q[:, :, sl_q], self.k[:, :, sl_k], self.v[:, :, sl_k], self.do[:, :, sl_q], self.out[:, :, sl_q],
                self.dk_acc[:, :, sl_k], self.dv_acc[:, :, sl_k])

    def forward(self):
        for r in range(self.W):
            q, k, v, _, out, _, _ = self._views(r)
            self.ops.attn_fwd(q, k, v, self.scale, True, r * self.Sc, out=out, lse=self.lse[r])

    def backward(self):
        """One launch pair (dQ, dK/dV) per rank, last rank first: its dK/dV launch covers every chunk and writes where
        the earlier ranks add, so no accumulator is cleared; delta = sum_d dO * O is computed inside the dQ kernel; dq is
        written in bf16 directly (a rank owns its query chunk), dk / dv are summed over the ranks in fp32."""
        ops = self.ops
        for r in reversed(range(self.W)):
            q, k, v, do, out, dk, dv = self._views(r)
            dq = self.dq_b[:, :, r * self.Sc:(r + 1) * self.Sc]
            ops.attn_bwd(do, q, k, v, self.lse[r], self.delta[r], self.scale, True, r * self.Sc, dq, dk, dv,
                         dkv_accumulate=r != self.W - 1, out=out)
        # hand the gradients back in the dtype of the inputs (autograd's cast in the reference)
        self.dk = ops.convert_f32(self.dk_acc, self.torch.bfloat16)
        self.dv = ops.convert_f32(self.dv_acc, self.torch.bfloat16)

    def step(self):
        self.forward()
        self.backward()

    def step_one_rank(self, r):
        """Forward + backward of cp rank r alone: its query chunk against chunks 0..r (one launch per direction)."""
        ops = self.ops
        q, k, v, do, out, dk, dv = self._views(r)
        ops.attn_fwd(q, k, v, self.scale, True, r * self.Sc, out=out, lse=self.lse[r])
        # (one block per rank in this schedule, so delta = sum_d dO * O is computed in the dQ kernel's prologue)
        ops.attn_bwd(do, q, k, v, self.lse[r], self.delta[r], self.scale, True, r * self.Sc, self.dq_acc[r], dk, dv,
                     dkv_accumulate=True, out=out)

    def step_one_rank_last_reader(self, r):
        """Forward + backward of cp rank r alone, with the gradient traffic that rank has in a real ring when it is the
        last rank to contribute to every chunk it reads (context_parallel.py:74-108 with is_causal: chunk c collects the
        blocks of ranks c, c+1, ... in that order, so the highest rank comes last): dq leaves in bf16; for the chunks of
        the ranks below, the fp32 sums that arrived with the chunk are read and the rounded total is written; the rank's
        own chunk, which nobody else reads, is written in bf16 directly.  One launch per direction over the chunk list."""
        ops, Sc = self.ops, self.Sc
        q, k, v, do, out, dk, dv = self._views(r)
        ks = [self.k[:, :, c * Sc:(c + 1) * Sc] for c in range(r + 1)]
        vs = [self.v[:, :, c * Sc:(c + 1) * Sc] for c in range(r + 1)]
        ops.attn_fwd_chunks(q, ks, vs, self.scale, True, r * Sc, out=out, lse=self.lse[r])
        sums_k = [self.dk_acc[:, :, c * Sc:(c + 1) * Sc] if c < r else None for c in range(r + 1)]
        sums_v = [self.dv_acc[:, :, c * Sc:(c + 1) * Sc] if c < r else None for c in range(r + 1)]
        ops.attn_bwd_chunks(do, q, ks, vs, self.lse[r], self.scale, True, r * Sc, self.dq_b[:, :, r * Sc:(r + 1) * Sc],
                            sums_k, sums_v, dkv_accumulate=[c < r for c in range(r + 1)], out=out, delta=self.delta[r],
                            dk_finals=[self.dk_b[:, :, c * Sc:(c + 1) * Sc] for c in range(r + 1)],
                            dv_finals=[self.dv_b[:, :, c * Sc:(c + 1) * Sc] for c in range(r + 1)])

    def step_ranks_parallel(self):
        """One launch per rank and direction, like step(), but the ranks' launches are independent branches: rank r's
        forward, delta pre-pass and dQ kernel run on stream r, the dK/dV launches (which add into shared chunks) follow
        each other on the calling stream, last rank first -- its launch covers every chunk and writes instead of adding,
        so no accumulator is cleared.  Recorded into a graph the streams become parallel branches of the graph."""
        torch, ops = self.torch, self.ops
        cur = torch.cuda.current_stream()
        if not hasattr(self, "_branch"):
            self._branch = [torch.cuda.Stream() for _ in range(self.W)]      # default priority
        ready = []
        for r, st in enumerate(self._branch):
            st.wait_stream(cur)
            with torch.cuda.stream(st):
                q, k, v, do, out, dk, dv = self._views(r)
                ops.attn_fwd(q, k, v, self.scale, True, r * self.Sc, out=out, lse=self.lse[r])
                ops.attn_bwd_preprocess(do, out, delta=self.delta[r])
                ev = torch.cuda.Event()
                ev.record(st)
                ready.append(ev)
                ops.attn_bwd(do, q, k, v, self.lse[r], self.delta[r], self.scale, True, r * self.Sc, self.dq_acc[r],
                             want_dkv=False)
        for r in reversed(range(self.W)):
            cur.wait_event(ready[r])
            q, k, v, do, out, dk, dv = self._views(r)
            ops.attn_bwd(do, q, k, v, self.lse[r], self.delta[r], self.scale, True, r * self.Sc, None, dk, dv,
                         dkv_accumulate=r != self.W - 1, want_dq=False)
        for st in self._branch:
            cur.wait_stream(st)
        self.dq = [ops.convert_f32(self.dq_acc[r], torch.bfloat16) for r in range(self.W)]
        self.dk = ops.convert_f32(self.dk_acc, torch.bfloat16)
        self.dv = ops.convert_f32(self.dv_acc, torch.bfloat16)

    # -- all four ranks in one launch per direction (q_offset 0 over the whole sequence)
    def forward_batched(self):
        self.ops.attn_fwd(self.q, self.k, self.v, self.scale, True, 0, out=self.out, lse=self.lse_b)

    def backward_kernel_batched(self):
        self.ops.attn_bwd(self.do, self.q, self.k, self.v, self.lse_b, self.delta_b, self.scale, True, 0, self.dq_b,
                          self.dk_b, self.dv_b)

    def backward_dkdv_only(self):
        self.ops.attn_bwd(self.do, self.q, self.k, self.v, self.lse_b, self.delta_b, self.scale, True, 0, None,
                          self.dk_b, self.dv_b, want_dq=False)

    def backward_dq_only(self):
        self.ops.attn_bwd(self.do, self.q, self.k, self.v, self.lse_b, self.delta_b, self.scale, True, 0, self.dq_b,
                          want_dkv=False)

    def step_batched(self):
        # forward, then the backward as one call: the dQ kernel computes delta = sum_d dO * O in its prologue and the
        # dK/dV kernel follows it
        self.forward_batched()
        self.ops.attn_bwd(self.do, self.q, self.k, self.v, self.lse_b, self.delta_b, self.scale, True, 0, self.dq_b,
                          self.dk_b, self.dv_b, out=self.out)

    # -- the same work in the reference's shape: one launch per ring step (block + fused merge)
    def step_per_ring_step(self):
        torch, ops, Sc = self.torch, self.ops, self.Sc
        self.dk_acc.zero_()
        self.dv_acc.zero_()
        for r in range(self.W):
            q = self.q[:, :, r * Sc:(r + 1) * Sc]
            do = self.do[:, :, r * Sc:(r + 1) * Sc]
            out32 = torch.empty(self.B, self.H, Sc, self.D, dtype=torch.float32, device=q.device)
            lse = self.lse[r]
            for s in range(r + 1):
                c = r - s
                ops.attn_fwd(q, self.k[:, :, c * Sc:(c + 1) * Sc], self.v[:, :, c * Sc:(c + 1) * Sc], self.scale, s == 0, 0,
                             out=out32, lse=lse, merge=s > 0)
            out = ops.convert_f32(out32, torch.bfloat16)
            delta = ops.attn_bwd_preprocess(do, out)
            for s in range(r + 1):
                c = r - s
                sl = slice(c * Sc, (c + 1) * Sc)
                ops.attn_bwd(do, q, self.k[:, :, sl], self.v[:, :, sl], lse, delta, self.scale, s == 0, 0, self.dq_acc[r],
                             self.dk_acc[:, :, sl], self.dv_acc[:, :, sl], dq_accumulate=s > 0, dkv_accumulate=True)
        self.dq = [ops.convert_f32(self.dq_acc[r], torch.bfloat16) for r in range(self.W)]
        self.dk = ops.convert_f32(self.dk_acc, torch.bfloat16)
        self.dv = ops.convert_f32(self.dv_acc, torch.bfloat16)


def ring_api_extra(torch, ops, rb, iters=20, eager_only=False):
    """The public API at configs[1]: ring_attention() (RingAttentionFunc, context_parallel.py:14-51) forward and
    backward for the four virtual cp ranks -- every rank's own q / k / v chunk tensors (leaves that require gradients),
    the ranks played in ascending order, one backward over all of them.  Autograd, the mailbox, the chunks' publishing
    nodes and the fp32 -> bf16 hand-back of dk / dv are all inside the timed region.  Timed as replays of a HIP graph of
    the whole step (what a captured training step pays) and as eager launches (bound by the host: Python + autograd
    per call)."""
    import picotron_amd.process_group_manager as pgm
    from picotron_amd.context_parallel import context_parallel as cp
    W, Sc = rb.W, rb.Sc
    mgr = pgm.setup_process_group_manager(1, W, 1, 1)
    leaves = [[t[:, :, r * Sc:(r + 1) * Sc].clone().requires_grad_() for t in (rb.q, rb.k, rb.v)] for r in range(W)]
    # the output gradient in the memory layout of the output ([B,S,H,D], as it arrives from the o_proj's backward through
    # the free transpose + reshape of model.py:160): a gradient laid out otherwise makes the backward copy `out` first
    dos = [rb.do[:, :, r * Sc:(r + 1) * Sc].transpose(1, 2).contiguous().transpose(1, 2) for r in range(W)]
    total_flops = sum(rb.flops())

    def step():
        # a new pass: the same leaf tensors come back every step, and without this the mailbox would take them for
        # chunks staged ahead and hand out the previous step's publishing nodes
        mgr.cp_ring.reset()
        outs = []
        for r in range(W):
            mgr.set_cp_rank(r)
            outs.append(cp.ring_attention(*leaves[r], rb.scale, True))
        torch.autograd.backward(outs, dos)

    def clear():
        for ts in leaves:
            for t in ts:
                t.grad = None

    res = {"what": "ring_attention() forward + backward over the 4 virtual ranks of configs[1] through autograd "
                   "(one launch per rank and direction over the chunk list; PICO_RING_PER_STEP=1 gives the per-step shape)"}
    try:
        if eager_only:
            raise RuntimeError("not asked for")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                clear()
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        clear()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        preheat(torch, graph.replay, 0.2)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            graph.replay()
        stop.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(stop) / iters
        res["graph_replay"] = {"ms_per_step": round(ms, 4), "TFLOP/s": round(total_flops / (ms * 1e-3) / 1e12, 2),
                               "frac_of_mfma_peak": round(total_flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
        del graph
    except Exception as e:   # a capture that the autograd engine or the allocator refuses: report it, keep the eager figure
        res["graph_replay"] = {"error": repr(e)[:200]}
        torch.cuda.synchronize()
    for _ in range(3):
        clear()
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        clear()
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / iters
    res["eager"] = {"ms_per_step": round(ms, 4), "TFLOP/s": round(total_flops / (ms * 1e-3) / 1e12, 2),
                    "note": "host-bound: Python, autograd and ctypes per call"}
    pgm.setup_process_group_manager(1, 1, 1, 1)
    return res


def seq_len_extra(torch, ops, iters=10):
    """The headline step (one causal forward + backward launch set over whole sequences, head_dim 64, 32 heads) at the
    same 4096 tokens but longer sequences: configs[1]'s launches are one generation of workgroups whose loads and stores
    are not hidden behind anyone's matrix work; with more trips per workgroup that share shrinks."""
    out = {}
    for B, S in ((4, 1024), (2, 2048), (1, 4096), (1, 8192)):
        rb = RingBench(torch, ops, B=B, S=S, W=1)
        fwd_flops, bwd_flops = rb.flops()
        ms, _ = graph_time(torch, rb.step_batched, iters, per_graph=5)
        out[f"B{B}_S{S}"] = {"ms_per_step": round(ms, 4), "TFLOP/s": round((fwd_flops + bwd_flops) / (ms * 1e-3) / 1e12, 1),
                            "frac_of_mfma_peak": round((fwd_flops + bwd_flops) / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
        del rb
    return out


def preheat(torch, launch, seconds=0.1, batch=10):
    """Untimed launches for `seconds` of wall-clock, ending on a synchronize.  The GPU's clocks follow its load with a
    delay: after an idle stretch (a graph capture, host-side set-up) the first tens of milliseconds of work run about
    10 % slower than the steady state, so every timed region starts right after one of these.  Returns the launches."""
    n, t0 = 0, time.perf_counter()
    while True:
        for _ in range(batch):
            launch()
        torch.cuda.synchronize()
        n += batch
        if time.perf_counter() - t0 >= seconds:
            return n


def graph_time(torch, fn, iters, warmup=3, per_graph=1):
    """Records fn() `per_graph` times into a HIP graph and returns (ms per fn() over `iters` replays, graph).
    Each replay is one graph launch, and the GPU idles for about 8 us between two of them; with several
    calls recorded per graph that gap is shared out, as it is in a training step recorded as one graph."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(warmup):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(per_graph):
            fn()
    preheat(torch, graph.replay, 0.2)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        graph.replay()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / (iters * per_graph), graph


def bandwidth_extras(torch, ops, iters=50):
    """RMSNorm / RoPE / SwiGLU at the SmolLM-1.7B step's sizes (T = 4096 tokens, h 2048, I 8192, 32 heads of 64).
    `cold` rotates over enough buffers to exceed the 256 MB Infinity Cache, `warm` reuses one set."""
    dev = "cuda"
    bf = torch.bfloat16
    T, h, I, B, H, S, D = 4096, 2048, 8192, 4, 32, 1024, 64
    res = {}

    def run(name, make, call, bytes_per_call, nsets_cold):
        for label, nsets in (("cold", nsets_cold), ("warm", 1)):
            sets = [make() for _ in range(nsets)]
            def body():
                for s_ in sets:
                    call(*s_)
            # the warm variant records ten calls per graph so that the idle time between graph launches is shared out
            ms, _ = graph_time(torch, body, iters, per_graph=10 if nsets == 1 else 1)
            gbs = bytes_per_call * nsets / (ms * 1e-3) / 1e9
            res[f"{name}_{label}"] = {"GB/s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 3),
                                      "us_per_call": round(ms * 1e3 / nsets, 2), "algorithmic_MB": round(bytes_per_call / 1e6, 2)}
            del sets

    # what the memory system gives a plain device-to-device copy of the same sizes (torch's copy kernel): the
    # practical ceiling for a read-once / write-once kernel at this size, well below the 8 TB/s pin rate
    run("copy_33MB_reference", lambda: (torch.randn(T, h, device=dev).to(bf), torch.empty(T, h, dtype=bf, device=dev)),
        lambda x, y: y.copy_(x), 2 * T * h * 2, 24)
    run("copy_201MB_reference", lambda: (torch.randn(T, 3 * I // 2, device=dev).to(bf), torch.empty(T, 3 * I // 2, dtype=bf, device=dev)),
        lambda x, y: y.copy_(x), 2 * T * (3 * I // 2) * 2, 4)
    w = torch.ones(h, dtype=bf, device=dev)
    run("rmsnorm_fwd", lambda: (torch.randn(T, h, device=dev).to(bf),),
        lambda x: ops.rmsnorm_fwd(x, w, 1e-5, False), 2 * T * h * 2 + h * 2, 24)
    rstd = torch.rand(T, device=dev) + 0.5
    run("rmsnorm_bwd", lambda: (torch.randn(T, h, device=dev).to(bf), torch.randn(T, h, device=dev).to(bf)),
        lambda dy, x: ops.rmsnorm_bwd(dy, x, w, rstd), 3 * T * h * 2 + h * 4, 16)
    cos = torch.rand(S, D, device=dev).to(bf)
    sin = torch.rand(S, D, device=dev).to(bf)
    run("rope", lambda: (torch.randn(B, S, H, D, device=dev).to(bf).transpose(1, 2),),
        lambda x: ops.rope(x, cos, sin), 2 * B * H * S * D * 2 + S * D * 2, 24)
    run("swiglu_fwd", lambda: (torch.randn(T, I, device=dev).to(bf), torch.randn(T, I, device=dev).to(bf)),
        lambda g_, u: ops.swiglu_fwd(g_, u), 3 * T * I * 2, 4)
    run("swiglu_bwd", lambda: tuple(torch.randn(T, I, device=dev).to(bf) for _ in range(3)),
        lambda dy, g_, u: ops.swiglu_bwd(dy, g_, u), 5 * T * I * 2, 3)
    # cross-entropy over the 49152-entry vocabulary of the step: forward reads the logits once, backward reads them
    # again and writes dlogits
    Vc = 49152
    tg = torch.randint(0, Vc, (T,), device=dev)
    one = torch.ones(1, device=dev)
    run("cross_entropy_fwd", lambda: (torch.randn(T, Vc, device=dev).to(bf),),
        lambda lg: ops.cross_entropy_fwd(lg, tg), T * Vc * 2, 2)
    lse_c = ops.cross_entropy_fwd(torch.randn(T, Vc, device=dev).to(bf), tg)[1]
    run("cross_entropy_bwd", lambda: (torch.randn(T, Vc, device=dev).to(bf),),
        lambda lg: ops.cross_entropy_bwd(lg, tg, lse_c, one), 2 * T * Vc * 2, 2)
    # AdamW on 256 Mi bf16 parameters: 28 bytes per parameter with fp32 master weights and moments, 22 with fp32 moments
    # only, 14 with bf16 state.  The working set (3.8-7.5 GB) is that of a real parameter list: on 64 Mi parameters
    # (1.5 GB) kernel variants that gain nothing on a model's optimizer step measured 11-16 % faster.
    n = 256 * 1024 * 1024
    run("adamw", lambda: (torch.zeros(n, device=dev, dtype=bf), torch.randn(n, device=dev), torch.randn(n, device=dev).to(bf),
                          torch.zeros(n, device=dev), torch.zeros(n, device=dev)),
        lambda p_, m_, g_, ea, eas: ops.adamw_(p_, m_, g_, ea, eas, 1, 1e-3), 28 * n, 1)
    run("adamw_lp_fp32_moments", lambda: (torch.randn(n, device=dev).to(bf), torch.randn(n, device=dev).to(bf), torch.randn(n, device=dev), torch.rand(n, device=dev)),
        lambda p_, g_, ea, eas: ops.adamw_lp_(p_, g_, ea, eas, 1, 1e-3), 22 * n, 1)
    run("adamw_lp_bf16_moments", lambda: tuple(torch.randn(n, device=dev).to(bf) for _ in range(3)) + (torch.rand(n, device=dev).to(bf),),
        lambda p_, g_, ea, eas: ops.adamw_lp_(p_, g_, ea, eas, 1, 1e-3), 14 * n, 1)
    return res


def train_step_extra(torch, which="smollm_1p7b", steps=10, warmup=3, adamw="fp32_moments"):
    """configs[2]: SmolLM-1.7B-shaped training step (24 layers, h 2048, 32 heads of 64, I 8192, V 49152), mbs 4, seq 1024;
    configs[3]: Llama-2-7B-shaped step (32 layers, h 4096, 32 heads of 128, I 11008, V 32000), mbs 1, seq 4096.
    bf16 parameters, random init, synthetic tokens.  adamw selects the optimizer's memory layout:
    "fp32_moments" (the named configuration: bf16 parameters updated in place, fp32 AdamW state), "fp32_master" (an
    fp32 master copy of every parameter as well) or "reference" (the state as the reference holds it, train.py:209:
    AdamW on the bf16 parameters, so bf16 moments)."""
    import torch.nn.functional as F

    import picotron_amd.process_group_manager as pgm
    from picotron_amd.model import Llama
    from picotron_amd.utils import (MI355X_BF16_DENSE_FLOPS, flops_per_token, get_num_params, llama2_7b_shape,
                                    smollm_1p7b_shape, synthetic_tokens)

    pgm.setup_process_group_manager(1, 1, 1, 1)
    os.environ["CONTEXT_PARALLEL"] = "0"
    mbs, seq = (4, 1024) if which == "smollm_1p7b" else (1, 4096)
    cfg = smollm_1p7b_shape(seq) if which == "smollm_1p7b" else llama2_7b_shape(seq)
    torch.manual_seed(42)
    with torch.device("cuda"):
        model = Llama(cfg)
    model = model.to(torch.bfloat16)
    # one fused pass over the whole parameter list, up to 48 tensors per launch (picotron_amd.optim.FusedAdamW)
    from picotron_amd.functional import cross_entropy
    from picotron_amd.optim import FusedAdamW
    layouts = {"fp32_moments": (dict(master_weights=False, state_dtype=torch.float32), "bf16 parameters updated in place, fp32 moments"),
               "fp32_master": (dict(master_weights=True), "fp32 master weights and moments"),
               "reference": (dict(master_weights=False), "bf16 moments, bf16 parameter updated in place (the reference's layout)")}
    opt = FusedAdamW(model.parameters(), lr=3e-4, overlap_with_backward=os.getenv("PICO_BENCH_OVERLAP", "0") == "1",
                     **layouts[adamw][0])
    ids, tgt = synthetic_tokens(cfg.vocab_size, mbs, seq, seed=0)
    ids, tgt = ids.cuda(), tgt.cuda()

    def step():
        opt.zero_grad()
        logits = model(input_ids=ids)
        loss = cross_entropy(logits.view(mbs * seq, -1), tgt.reshape(-1))
        loss.backward()
        opt.step()
        return loss

    # the loss of the very first step (random init, nothing updated yet) is a function of the seed and the kernels
    # alone: reproducible to ~1e-2 across builds and close to ln(vocab); the loss after a dozen bf16 updates on one
    # batch is not (it differs by +-1 between builds), so it is not reported
    first_loss = None
    for _ in range(warmup):
        loss = step()
        if first_loss is None:
            first_loss = loss.item()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    n = get_num_params(model)
    tok_s = mbs * seq / dt
    fpt = flops_per_token(n, cfg.num_hidden_layers, cfg.hidden_size, seq)
    res = {"tokens_per_s": round(tok_s, 1), "ms_per_step": round(dt * 1e3, 2), "params": n, "loss_first_step": round(first_loss, 4),
           "ln_vocab": round(math.log(cfg.vocab_size), 4),
           "mfu_vs_2.5PF": round(tok_s * fpt / MI355X_BF16_DENSE_FLOPS, 4), "steps": steps,
           "adamw_state": layouts[adamw][1],
           "note": "attention / RMSNorm with the residual adds / RoPE / SwiGLU / cross-entropy / AdamW on the HIP kernels; "
                   "embedding and projections on torch"}
    del model, opt
    torch.cuda.empty_cache()
    return res


def long_context_extra(torch, ops, iters=10):
    """configs[4]: rank 7 of cp 8 at total seq 32768 -- 4096 queries over 8 K/V chunks of 4096, GQA 32/8, head_dim 128,
    forward + backward; 7.5 chunk-blocks of 14 * Hq * Sc^2 * D FLOP each = 7.215 TFLOP."""
    W, Sc, Hq, Hkv, D, r = 8, 4096, 32, 8, 128, 7
    scale = 1.0 / math.sqrt(D)
    g = torch.Generator().manual_seed(0)
    q = (torch.randn(1, Hq, Sc, D, generator=g) * scale).to(torch.bfloat16).cuda()
    k, v = (torch.randn(1, Hkv, W * Sc, D, generator=g).to(torch.bfloat16).cuda() for _ in range(2))
    do = torch.randn(1, Hq, Sc, D, generator=g).to(torch.bfloat16).cuda()
    out = torch.empty_like(q)
    lse = torch.empty(1, Hq, Sc, dtype=torch.float32, device="cuda")
    delta = torch.empty_like(lse)
    dq = torch.empty_like(q)
    dk, dv = torch.empty_like(k), torch.empty_like(v)
    flops = 7.5 * 14 * Hq * Sc * Sc * D

    def fused():
        ops.attn_fwd(q, k, v, scale, True, r * Sc, out=out, lse=lse)
        ops.attn_bwd_preprocess(do, out, delta=delta)
        ops.attn_bwd(do, q, k, v, lse, delta, scale, True, r * Sc, dq, dk, dv)

    o32 = torch.empty(1, Hq, Sc, D, dtype=torch.float32, device="cuda")
    dq32 = torch.empty_like(o32)
    dk32 = torch.empty(1, Hkv, W * Sc, D, dtype=torch.float32, device="cuda")
    dv32 = torch.empty_like(dk32)

    def per_ring_step():
        dk32.zero_()
        dv32.zero_()
        for s_ in range(W):
            cs = slice((r - s_) * Sc, (r - s_ + 1) * Sc)
            ops.attn_fwd(q, k[:, :, cs], v[:, :, cs], scale, s_ == 0, 0, out=o32, lse=lse, merge=s_ > 0)
        ob = ops.convert_f32(o32, torch.bfloat16)
        ops.attn_bwd_preprocess(do, ob, delta=delta)
        for s_ in range(W):
            cs = slice((r - s_) * Sc, (r - s_ + 1) * Sc)
            ops.attn_bwd(do, q, k[:, :, cs], v[:, :, cs], lse, delta, scale, s_ == 0, 0, dq32, dk32[:, :, cs], dv32[:, :, cs],
                         dq_accumulate=s_ > 0, dkv_accumulate=True)

    ms_f, _ = graph_time(torch, fused, iters)
    ms_r, _ = graph_time(torch, per_ring_step, iters)
    res = {"flops": flops, "one_launch_per_direction": {"ms": round(ms_f, 3), "TFLOP/s": round(flops / (ms_f * 1e-3) / 1e12, 1)},
           "one_launch_per_ring_step": {"ms": round(ms_r, 3), "TFLOP/s": round(flops / (ms_r * 1e-3) / 1e12, 1)}}

    # The rank's step as the ring runs it, RoPE included ("RoPE applied with absolute position ids offset by chunk
    # index"): K / V are the eight chunk tensors of the ranks (separate allocations; ranks 0..6 arrive rotated), rank 7
    # rotates its own k chunk (one launch), q is rotated inside the forward at positions 7 * 4096 + row, and the
    # backward un-rotates dq and dk of every chunk in its epilogues; dq in bf16, dk / dv of the chunks in fp32 (the
    # ring's travelling accumulators).  One launch per direction over the chunk list.
    from picotron_amd.model import get_cos_sin
    cos, sin = get_cos_sin(W * Sc, D, 10000.0)
    cos, sin = cos.cuda(), sin.cuda()
    k_raw = [k[:, :, c * Sc:(c + 1) * Sc].clone() for c in range(W)]
    v_ch = [v[:, :, c * Sc:(c + 1) * Sc].clone() for c in range(W)]
    k_rot = [ops.rope(k_raw[c], cos, sin, pos_offset=c * Sc) for c in range(W)]
    dk_ch = [torch.empty(1, Hkv, Sc, D, dtype=torch.float32, device="cuda") for _ in range(W)]
    dv_ch = [torch.empty(1, Hkv, Sc, D, dtype=torch.float32, device="cuda") for _ in range(W)]

    def with_rope():
        ops.rope(k_raw[r], cos, sin, pos_offset=r * Sc, out=k_rot[r])
        o, l, q_rot = ops.attn_fwd_chunks(q, k_rot, v_ch, scale, True, r * Sc, rope=(cos, sin), q_pos_offset=r * Sc, want_q_rot=True)
        ops.attn_bwd_chunks(do, q_rot, k_rot, v_ch, l, scale, True, r * Sc, dq, dk_ch, dv_ch, out=o, rope=(cos, sin),
                            q_pos_offset=r * Sc, k_pos_offset=0)

    ms_w, _ = graph_time(torch, with_rope, iters)
    res["one_launch_per_direction_rope_inside_chunk_list"] = {
        "ms": round(ms_w, 3), "TFLOP/s": round(flops / (ms_w * 1e-3) / 1e12, 1),
        "note": "k of the rank's own chunk rotated by one launch, q inside the forward, dq / dk un-rotated inside the backward; "
                "K / V as 8 separate chunk tensors, dk / dv per chunk in fp32"}
    del k_raw, v_ch, k_rot, dk_ch, dv_ch

    # RoPE at the rank's absolute positions (r * Sc + arange(Sc)): the q chunk and one K chunk, tables of the whole
    # sequence, pos_offset instead of sliced tables
    q_rot = torch.empty_like(q)
    k_rot = torch.empty_like(k[:, :, :Sc])
    ms_q, _ = graph_time(torch, lambda: ops.rope(q, cos, sin, pos_offset=r * Sc, out=q_rot), 20, per_graph=10)
    ms_k, _ = graph_time(torch, lambda: ops.rope(k[:, :, r * Sc:], cos, sin, pos_offset=r * Sc, out=k_rot), 20, per_graph=10)
    bytes_q, bytes_k = 2 * q.numel() * 2 + Sc * D * 2, 2 * k_rot.numel() * 2 + Sc * D * 2
    res["rope_at_offset_positions"] = {"q_chunk": {"us": round(ms_q * 1e3, 2), "GB/s": round(bytes_q / (ms_q * 1e-3) / 1e9, 1), "bytes": bytes_q},
                                       "k_chunk": {"us": round(ms_k * 1e3, 2), "GB/s": round(bytes_k / (ms_k * 1e-3) / 1e9, 1), "bytes": bytes_k},
                                       "note": "warm (same buffers every launch; 64 MiB and 16 MiB of traffic)"}

    # the reference's layout: K / V expanded to the query heads by repeat_interleave before attention; the kernels then
    # see 32 kv heads (4 x the K / V traffic and dK / dV of 32 heads)
    del o32, dq32, dk32, dv32, dk, dv
    group = Hq // Hkv
    ke, ve = k.repeat_interleave(group, dim=1), v.repeat_interleave(group, dim=1)
    dke, dve = torch.empty_like(ke), torch.empty_like(ve)

    def expanded():
        ops.attn_fwd(q, ke, ve, scale, True, r * Sc, out=out, lse=lse)
        ops.attn_bwd_preprocess(do, out, delta=delta)
        ops.attn_bwd(do, q, ke, ve, lse, delta, scale, True, r * Sc, dq, dke, dve)

    ms_e, _ = graph_time(torch, expanded, iters)
    res["pre_expanded_kv_heads"] = {"ms": round(ms_e, 3), "TFLOP/s": round(flops / (ms_e * 1e-3) / 1e12, 1)}
    return res


def cpu_baseline(host_tensors, W, scale, flops_total):
    """The CPU oracle on the same inputs: full configs[1] shape, fp32, all host threads and one thread."""
    import torch
    from oracle import ring
    q, k, v, do = (t.float() for t in host_tensors)
    out = {}
    cores = min(os.cpu_count() or 1, 16)
    for label, threads, reps in (("all_threads", cores, 4), ("one_thread", 1, 1)):
        torch.set_num_threads(threads)
        ring.all_ranks_forward(q[:1], k[:1], v[:1], W, scale, True)  # warm the allocator
        t0 = time.perf_counter()
        for _ in range(reps):
            o, l = ring.all_ranks_forward(q, k, v, W, scale, True)
            ring.all_ranks_backward(do, q, k, v, o, l, W, scale, True)
        dt = (time.perf_counter() - t0) / reps
        out[label] = {"value": round(flops_total / dt / 1e12, 5), "unit": "TFLOP/s", "cores": threads, "s_per_step": round(dt, 3)}
    torch.set_num_threads(cores)
    return out


def cpu_long_context_sample(threads):
    """configs[4] on the CPU oracle, bounded: one dense and one causal chunk-block (4096 x 4096, head_dim 128) for 4 of
    the 32 query heads (one kv head, expanded as the reference does), forward + backward in fp32; rank 7's 7 dense + 1
    causal blocks of 32 heads are extrapolated from it (x 8 heads-wise) and labelled as such."""
    import torch
    from oracle import ring
    torch.set_num_threads(threads)
    Sc, D, Hs = 4096, 128, 4
    scale = 1.0 / math.sqrt(D)
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, Hs, Sc, D, generator=g) * scale
    k, v, do = (torch.randn(1, Hs, Sc, D, generator=g) for _ in range(3))
    secs = {}
    for name, causal in (("dense", False), ("causal", True)):
        t0 = time.perf_counter()
        o, l = ring.block_forward(q, k, v, scale, causal)
        ring.block_backward(do, q, k, v, o, l, scale, causal)
        secs[name] = time.perf_counter() - t0
    rank_s = (7 * secs["dense"] + secs["causal"]) * (32 / Hs)
    flops = 7.5 * 14 * 32 * Sc * Sc * D
    return {"s_dense_block_4_heads": round(secs["dense"], 3), "s_causal_block_4_heads": round(secs["causal"], 3),
            "s_rank7_extrapolated": round(rank_s, 1), "TFLOP/s_extrapolated": round(flops / rank_s / 1e12, 4), "cores": threads,
            "what": "configs[4]: one dense + one causal 4096x4096 block of 4 query heads on the CPU oracle (fp32), "
                    "extrapolated to rank 7's 7 dense + 1 causal blocks of 32 heads"}


def cpu_configs0_step(threads):
    """configs[0], the reference's own CPU-runnable case, on the CPU oracle: SmolLM-135M-shaped model cut to 2 layers,
    fp32, B 2, S 256, one full training step (forward, CE, backward, AdamW); seconds per step after one warm-up step."""
    import torch
    from oracle.model import OracleLlama, smollm_135m_2layer, synthetic_batch, train_step
    torch.set_num_threads(threads)
    torch.manual_seed(42)
    cfg = smollm_135m_2layer(256)
    model = OracleLlama(cfg)
    opt = torch.optim.AdamW(model.parameters(), lr=3e-4)
    ids, tgt = synthetic_batch(cfg.vocab_size, 2, 256, seed=0)
    train_step(model, opt, ids, tgt)
    t0 = time.perf_counter()
    for _ in range(2):
        train_step(model, opt, ids, tgt)
    return (time.perf_counter() - t0) / 2


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this build has no multi-GPU path (asked for --gpus {args.gpus}); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from picotron_amd import ops
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    ops._lib.lib()  # fail loudly now if the HIP library is not built

    if args.train_step:
        print(json.dumps({args.train_step + "_train_step": train_step_extra(torch, args.train_step, steps=4, warmup=2)}))
        return
    if args.probe == "configs4":
        W, Sc, Hq, Hkv, D, r = 8, 4096, 32, 8, 128, 7
        scale = 1.0 / math.sqrt(D)
        g = torch.Generator().manual_seed(0)
        q = (torch.randn(1, Hq, Sc, D, generator=g) * scale).to(torch.bfloat16).cuda()
        k, v = (torch.randn(1, Hkv, W * Sc, D, generator=g).to(torch.bfloat16).cuda() for _ in range(2))
        do = torch.randn(1, Hq, Sc, D, generator=g).to(torch.bfloat16).cuda()
        out, dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        lse = torch.empty(1, Hq, Sc, dtype=torch.float32, device="cuda")
        src = torch.randn(16, 1024, 1024, dtype=torch.float32, device="cuda").view(1, 16, 1024, 1024)
        for _ in range(3):
            ops.convert_f32(src, torch.float32)
        for _ in range(3):
            ops.attn_fwd(q, k, v, scale, True, r * Sc, out=out, lse=lse)
            delta = ops.attn_bwd_preprocess(do, out)
            ops.attn_bwd(do, q, k, v, lse, delta, scale, True, r * Sc, None, dk, dv, want_dq=False)
            ops.attn_bwd(do, q, k, v, lse, delta, scale, True, r * Sc, dq, want_dkv=False)
        torch.cuda.synchronize()
        print(json.dumps({"probe": "convert_kernel<float> copies 67108864 B in and out per launch; attention kernels at configs[4] "
                                   "(rank 7 of 8: 4096 queries x 32768 keys, GQA 32/8, head_dim 128)"}))
        return
    rb = RingBench(torch, ops)
    if args.probe == "ring_api":
        # the public API's step (ring_attention() forward + backward over the four virtual ranks), launched eagerly a few
        # times so that a kernel trace shows what one step consists of
        res = ring_api_extra(torch, ops, rb, iters=20, eager_only=True)
        print(json.dumps({"probe": "ring_attention() through autograd over the 4 virtual ranks of configs[1], eager", **res["eager"]}))
        return
    if args.probe:
        # plain copy of 64 MiB fp32 (read 64 MiB, write 64 MiB) as the scale for the HBM counters
        src = torch.randn(16, 1024, 1024, dtype=torch.float32, device="cuda").view(1, 16, 1024, 1024)
        for _ in range(5):
            ops.convert_f32(src, torch.float32)
        rb.forward_batched()
        ops.attn_bwd_preprocess(rb.do, rb.out, delta=rb.delta_b)
        for _ in range(5):
            rb.forward_batched()
            rb.backward_dkdv_only()
            rb.backward_dq_only()
        torch.cuda.synchronize()
        print(json.dumps({"probe": "convert_kernel<float> copies 67108864 B in and out per launch; attention kernels at configs[1]"}))
        return
    fwd_flops, bwd_flops = rb.flops()
    total_flops = fwd_flops + bwd_flops

    # ---- W warm-up steps, then EXACTLY K timed steps, twice: as replays of a HIP graph of the step and as plain stream
    #      launches; each timed region follows 100 ms of the same launches untimed (see preheat).  `value` is the faster.
    for _ in range(max(args.warmup, 1)):
        rb.step_batched()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        rb.step_batched()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    # several steps are recorded per graph (the largest divisor of K up to 20) so that exactly K steps are timed and
    # the idle time between two graph launches is not charged to every single step
    per_graph = max(g for g in range(1, 21) if args.steps % g == 0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(per_graph):
            rb.step_batched()
    preheat_steps = preheat(torch, graph.replay, 0.1, batch=2) * per_graph
    t0 = time.perf_counter()
    for _ in range(args.steps // per_graph):
        graph.replay()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_graph = (t1 - t0) * 1e3 / args.steps
    preheat_steps = max(preheat_steps, preheat(torch, rb.step_batched, 0.1, batch=50))
    t0 = time.perf_counter()
    for _ in range(args.steps):
        rb.step_batched()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_eager = (t1 - t0) * 1e3 / args.steps
    ms_per_step = min(ms_graph, ms_eager)
    value = total_flops / (ms_per_step * 1e-3) / 1e12

    # ---- dominant kernel: the dK/dV launch alone, HIP events on the launching stream.  Its algorithmic work
    #      is 4 of the backward's 5 matrix products (S, dP, dV, dK): 8 FLOPs per (query, key, d) triple.
    dkdv_flops = bwd_flops * 0.8
    # (median of three measurements: a single one was once seen 50 % high on an otherwise normal run)
    ms_dkdv = sorted(graph_time(torch, rb.backward_dkdv_only, max(args.steps // 10, 10), per_graph=10)[0] for _ in range(3))[1]
    dkdv_tflops = dkdv_flops / (ms_dkdv * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": "attn_bwd_dkdv_kernel_d64", "achieved": round(dkdv_tflops, 2),
                "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(dkdv_tflops / MFMA_BF16_PEAK_TFLOPS, 4),
                "avg_launch_us": round(ms_dkdv * 1e3, 2), "flops_per_launch": dkdv_flops, "traffic": TRAFFIC_BYTES_DKDV}

    extras = {}
    if not args.no_extras:
        ms_dq, _ = graph_time(torch, rb.backward_dq_only, max(args.steps // 10, 10), per_graph=10)
        ms_bwd_k, _ = graph_time(torch, rb.backward_kernel_batched, max(args.steps // 10, 10), per_graph=10)
        extras["attn_bwd_dq_kernel"] = {"us_per_launch": round(ms_dq * 1e3, 2),
                                        "TFLOP/s_algorithmic": round(bwd_flops * 0.2 / (ms_dq * 1e-3) / 1e12, 2),
                                        "TFLOP/s_executed": round(bwd_flops * 0.6 / (ms_dq * 1e-3) / 1e12, 2),
                                        "note": "recomputes S and dP: executes 3 products for 1 algorithmic"}
        extras["attn_bwd_both_kernels"] = {"us": round(ms_bwd_k * 1e3, 2), "TFLOP/s_algorithmic": round(bwd_flops / (ms_bwd_k * 1e-3) / 1e12, 2)}
        ms_fwd, _ = graph_time(torch, rb.forward_batched, max(args.steps // 10, 10), per_graph=10)
        extras["attn_fwd_kernel"] = {"TFLOP/s": round(fwd_flops / (ms_fwd * 1e-3) / 1e12, 2), "us_per_launch": round(ms_fwd * 1e3, 2),
                                     "frac_of_mfma_peak": round(fwd_flops / (ms_fwd * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
        ms_rank, _ = graph_time(torch, rb.step, max(args.steps // 4, 10))
        extras["one_launch_per_rank"] = {"TFLOP/s": round(total_flops / (ms_rank * 1e-3) / 1e12, 2), "ms_per_step": round(ms_rank, 4),
                                         "frac_of_mfma_peak": round(total_flops / (ms_rank * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                                         "schedule": "ranks one after another on one stream"}
        ms_par, _ = graph_time(torch, rb.step_ranks_parallel, max(args.steps // 4, 10))
        extras["one_launch_per_rank_parallel_branches"] = {
            "TFLOP/s": round(total_flops / (ms_par * 1e-3) / 1e12, 2), "ms_per_step": round(ms_par, 4),
            "frac_of_mfma_peak": round(total_flops / (ms_par * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
            "schedule": "rank r's forward, delta and dQ on graph branch r; the dK/dV launches in sequence, last rank first"}
        ms_r3, _ = graph_time(torch, lambda: rb.step_one_rank(3), max(args.steps // 10, 10), per_graph=10)
        r3_flops = total_flops * 3.5 / 8.0   # 1 causal + 3 dense chunk-blocks of the 8 block-equivalents of all ranks
        extras["rank3_of_4_alone"] = {"TFLOP/s": round(r3_flops / (ms_r3 * 1e-3) / 1e12, 2), "us_per_step": round(ms_r3 * 1e3, 2),
                                      "flops": r3_flops,
                                      "frac_of_mfma_peak": round(r3_flops / (ms_r3 * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                                      "schedule": "the last rank's share alone: 256 queries of every head over chunks 0..3; fp32 dq, "
                                                  "fp32 dk / dv sums of all four chunks read, added to and written back"}
        ms_r3l, _ = graph_time(torch, lambda: rb.step_one_rank_last_reader(3), max(args.steps // 10, 10), per_graph=10)
        extras["rank3_of_4_alone_as_last_reader"] = {
            "TFLOP/s": round(r3_flops / (ms_r3l * 1e-3) / 1e12, 2), "us_per_step": round(ms_r3l * 1e3, 2),
            "frac_of_mfma_peak": round(r3_flops / (ms_r3l * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
            "schedule": "the same share with the gradient traffic rank 3 has in the ring, where it contributes last to every chunk: "
                        "bf16 dq; fp32 sums of chunks 0..2 read and their rounded totals written; its own chunk written in bf16"}
        extras["ring_attention_api"] = ring_api_extra(torch, ops, rb)
        ms_ring, _ = graph_time(torch, rb.step_per_ring_step, max(args.steps // 4, 10))
        extras["one_launch_per_ring_step"] = {"TFLOP/s": round(total_flops / (ms_ring * 1e-3) / 1e12, 2), "ms_per_step": round(ms_ring, 4),
                                              "frac_of_mfma_peak": round(total_flops / (ms_ring * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                                              "schedule": "the reference's shape: block + fused merge per ring step, ranks and steps in sequence"}
        extras["same_step_at_longer_sequences"] = seq_len_extra(torch, ops)
        extras["bandwidth_kernels"] = bandwidth_extras(torch, ops)
        extras["configs4_long_context_rank7_of_8"] = long_context_extra(torch, ops)
        if not args.no_train:
            extras["smollm_1p7b_train_step"] = train_step_extra(torch, "smollm_1p7b")
            extras["smollm_1p7b_train_step_fp32_master"] = train_step_extra(torch, "smollm_1p7b", adamw="fp32_master")
            extras["smollm_1p7b_train_step_reference_adamw_layout"] = train_step_extra(torch, "smollm_1p7b", adamw="reference")
            extras["llama2_7b_train_step"] = train_step_extra(torch, "llama2_7b")

    line = {
        "metric": "causal ring-attn fwd+bwd TFLOP/s", "value": round(value, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[1]: causal ring attention fwd+bwd, B4 H32 S1024 D64, cp_size 4, the ring steps of all "
                               "4 ranks on one GPU (ranks batched into one launch per direction)",
                   "global_batch": 4, "seq_len": 1024, "flops_per_step": total_flops, "launch": "stream launches" if ms_eager <= ms_graph else "hip graph replays",
                   "ms_per_step_stream_launches": round(ms_eager, 4), "ms_per_step_graph_replays": round(ms_graph, 4),
                   "steps_per_graph_launch": per_graph, "untimed_preheat_steps": preheat_steps},
        "frac_of_mfma_peak": round(value / MFMA_BF16_PEAK_TFLOPS, 4),
        "roofline": roofline,
    }
    if not args.no_cpu:
        cpu = cpu_baseline(rb.host, rb.W, rb.scale, total_flops)
        main_leg = cpu["all_threads"]
        line["cpu_baseline"] = {"value": main_leg["value"], "unit": "TFLOP/s", "cores": main_leg["cores"], "kind": "port",
                                "sample": f"full configs[1] shape (fwd+bwd of all 4 ranks), fp32, {main_leg['s_per_step']} s per step; "
                                          f"one thread: {cpu['one_thread']['value']} TFLOP/s ({cpu['one_thread']['s_per_step']} s per step)"}
        c0_all, c0_one = cpu_configs0_step(main_leg["cores"]), cpu_configs0_step(1)
        line["cpu_baseline"]["configs0_step"] = {"tokens_per_s_all_threads": round(512 / c0_all, 1), "s_per_step_all_threads": round(c0_all, 3),
                                                 "tokens_per_s_one_thread": round(512 / c0_one, 1), "s_per_step_one_thread": round(c0_one, 3),
                                                 "what": "configs[0]: 2-layer SmolLM-135M shape, fp32, B2 S256, full training step on the CPU oracle"}
        line["cpu_baseline"]["configs4_sample"] = cpu_long_context_sample(main_leg["cores"])
    if extras:
        line["extras"] = extras
    print(json.dumps(line))


if __name__ == "__main__":
    main()
