#!/usr/bin/env python3
"""
Benchmark of the NativeLstm2 forward hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

Workload (default): benchmark configuration cfg3 (returnn_amd/synthetic.py), the bidirectional pair at n=1024 -- T=1000, B=32, bf16 weights and
activations with fp32 accumulate and cell state, ragged lengths in [500,1000]; one step = two op calls on
the same inputs (step=+1 and step=-1), issued through the C ABI with inputs, outputs and workspace already
resident in HBM.  ``value`` = timesteps x sequences processed per second = 2*T*B*K / elapsed (padded frames
counted, both directions).

Prints ONE JSON line with the throughput, a ``roofline`` object for the dominant kernel (the persistent
step kernel; algorithmic GEMM flops 8*T*B*n^2 per launch over the HIP-event duration of a call on the launch
stream) and a ``cpu_baseline`` object (the CPU restatement of the reference's path -- per-step BLAS SGEMM plus
the sequential pointwise loop -- timed on this host on a bounded sample of the same shape in fp32).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

_root = os.path.dirname(os.path.abspath(__file__))
if _root not in sys.path:
    sys.path.insert(0, _root)

PEAK_MFMA = {"bf16": 2.5e15, "f32": 157.3e12}  # MI355X dense matrix peaks, FLOP/s
PEAK_HBM = 8.0e12  # B/s

# HBM bytes per launch of the dominant kernel are not measured by this script: they come from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE runs of this same command (each counter scaled by what it reads for a plain 1 GiB device copy), whose
# summaries sit under profiles/.  profiles/hbm_traffic_per_launch.json lists them by workload, launches per step and
# plan text; a run whose plan is not in the list reports no traffic figure rather than somebody else's.
def copy_calibration(args, dev):
    """A plain device copy of known size before the timed region (``--copy-calibration-mib``): what FETCH_SIZE and
    WRITE_SIZE read for it scales the counters of the kernels of interest in a profile of the same run."""
    if args.copy_calibration_mib > 0:
        import torch

        src = torch.empty((args.copy_calibration_mib << 20,), dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads and writes copy_calibration_mib MiB each
        torch.cuda.synchronize()
        del src, dst


def measured_traffic(workload: str, launches: int, plan: str):
    """-> (bytes per launch or None, the profile summary the figure is transcribed from or None)"""
    path = os.path.join(_root, "profiles", "hbm_traffic_per_launch.json")
    try:
        with open(path) as f:
            entries = json.load(f)["entries"]
    except (OSError, ValueError, KeyError):
        return None, None
    key = plan.split(" launches=")[0]
    for e in entries:
        if e.get("workload") == workload and e.get("launches_per_step") == launches and e.get("plan") == key:
            return float(e["bytes_per_launch"]), e.get("source")
    return None, None


def algorithmic_bytes_per_unit(n: int, dtype: str) -> int:
    """HBM bytes per timestep x sequence: read X (4n), write H (4n), Y (n) in the activation type,
    write C (n, fp32), read the mask (4 bytes)."""
    e = 2 if dtype == "bf16" else 4
    return e * 4 * n + e * 4 * n + e * n + 4 * n + 4


def ceiling_fields(probe_us, seq_ms, issue_ms, rows, n, dtype, T, call_ms):
    """
    Three ceilings of the recurrent GEMM next to the nominal matrix peak.

    ``achievable_mfma``: the rate at which the device's matrix cores run the plan's per-workgroup MFMA tile sequence
    when nothing else happens (``issue_ms``: one launch of the library's issue probe -- the plan's grid, W and the
    hidden-state fragments in registers, per step the plan's MFMAs and nothing else: no LDS, no barrier, no loads),
    counted in the op's algorithmic flops.  This is the "achievable MFMA roofline" of the tile sequence;
    ``frac_of_achievable_mfma`` = issue-probe time / measured time.

    ``decomposition_ceiling``: the same with what the split of the contraction over four wavefronts adds
    (``seq_ms``: the sequence probe -- B fragments from LDS, the MFMAs, the partial tiles through LDS with the step's
    one barrier, their sum; no exchange, no streams, no gates): the best a kernel of this decomposition could do if the
    hidden state cost nothing to hand over.  ``frac_of_decomposition_ceiling`` = sequence-probe time / measured time.

    ``latency_ceiling``: the T steps are sequential, and a step cannot be shorter than one hand-over of the hidden state
    between the CUs that hold W (``probe_us``: the library's latency probe -- device-scope store, visible on every CU,
    device-scope load, at a tiny volume) plus the time the whole chip's matrix cores need for the step's GEMM at their
    peak.  A latency bound, not a roofline: the rate at that bound and ``frac_of_latency_ceiling`` say how far the
    kernel is from a perfect hand-over.
    """
    out = {}
    step_flops = 8.0 * n * n * rows
    if issue_ms is not None:
        out.update({
            "mfma_issue_us_per_step": issue_ms * 1e3 / T,
            "achievable_mfma": step_flops * T / (issue_ms * 1e-3) / 1e12,
            "frac_of_achievable_mfma": issue_ms / call_ms,
        })
    if seq_ms is not None:
        out.update({
            "mfma_sequence_us_per_step": seq_ms * 1e3 / T,
            "decomposition_ceiling": step_flops * T / (seq_ms * 1e-3) / 1e12,
            "frac_of_decomposition_ceiling": seq_ms / call_ms,
        })
    if probe_us is not None:
        mfma_us = step_flops / PEAK_MFMA[dtype] * 1e6
        ceiling_ms = (probe_us + mfma_us) * T * 1e-3
        out.update({
            "handover_latency_us": probe_us,
            "mfma_peak_us_per_step": mfma_us,
            "latency_ceiling": step_flops * T / (ceiling_ms * 1e-3) / 1e12,
            "frac_of_latency_ceiling": ceiling_ms / call_ms,
        })
    return out


def step_budget(call_ms, nowait_ms, seq_ms, issue_ms, T):
    """
    Where a time step of the persistent kernel goes, from four launches of T steps each timed in this run; the entries
    add up to the measured step by construction, each is the difference of two measurements:

    * ``mfma_issue``: the issue probe (the plan's MFMAs per wavefront and nothing else);
    * ``partial_tiles_through_lds``: sequence probe - issue probe (what the decomposition adds to the bare MFMAs: B
      operands made ready in front of them, the matrix pipeline running empty before the four wavefronts' partial tiles
      can be written to LDS, the step's barrier, their sum read back);
    * ``gates_streams_stores``: the op's kernel with the reads of the hidden state switched off - sequence probe (gate
      arithmetic, cell update, the exchange stores, what the X / H / Y / C streams cost although they ride behind the
      MFMAs);
    * ``exchange_wait``: the op's kernel - the same with those reads switched off (the delay in front of the first read
      of the hidden state, the read's round trip through L2, its check, repeated reads).
    """
    if None in (call_ms, nowait_ms, seq_ms, issue_ms):
        return None
    us = lambda ms: ms * 1e3 / T  # noqa: E731
    return {
        "mfma_issue": us(issue_ms),
        "partial_tiles_through_lds": us(seq_ms - issue_ms),
        "gates_streams_stores": us(nowait_ms - seq_ms),
        "exchange_wait": us(call_ms - nowait_ms),
        "sum": us(call_ms),
        "no_wait_launch_ms": nowait_ms,
    }


def blas_thread_count():
    """Threads the BLAS behind numpy uses for one SGEMM, and where that figure comes from."""
    try:
        from threadpoolctl import threadpool_info

        counts = [int(i.get("num_threads", 1)) for i in threadpool_info() if i.get("user_api") == "blas"]
        if counts:
            return max(counts), "threadpoolctl (threads of the BLAS that numpy links)"
    except Exception:
        pass
    if os.environ.get("OMP_NUM_THREADS"):
        return int(os.environ["OMP_NUM_THREADS"]), "OMP_NUM_THREADS"
    return int(os.cpu_count() or 1), "os.cpu_count()"


def cpu_baseline(name: str, target_seconds: float = 15.0):
    """Times the CPU restatement (test infrastructure, used here only as the reported baseline): on all BLAS threads
    (``value``) and, on a fifth of the time budget, on one thread (``value_1thread``; the reference's tests pin one
    thread, tests/_set_num_threads1.py)."""
    import contextlib

    from oracle import lstm2_oracle
    from returnn_amd import synthetic

    blas_threads, source = blas_thread_count()
    full_T = synthetic.make_config.__globals__["_SPECS"][name]["T"]

    def timed(seconds):
        probe_T = 25
        p = synthetic.make_config(name, T=probe_T)
        lstm2_oracle.native_lstm2_fwd_blas(p.X[:2], p.W, p.y0, p.c0, p.i[:2])  # warm-up (BLAS thread pool, page-in)
        t0 = time.perf_counter()
        lstm2_oracle.native_lstm2_fwd_blas(p.X, p.W, p.y0, p.c0, p.i)
        per_frame = (time.perf_counter() - t0) / probe_T
        T = int(max(probe_T, min(full_T, seconds / max(per_frame, 1e-9))))
        p = synthetic.make_config(name, T=T)
        reps = int(max(1, min(50, round(seconds / max(per_frame * T, 1e-9)))))
        t0 = time.perf_counter()
        for _ in range(reps):
            lstm2_oracle.native_lstm2_fwd_blas(p.X, p.W, p.y0, p.c0, p.i)
        dt = time.perf_counter() - t0
        return reps * p.T * p.B / dt, p, reps, dt

    value, p, reps, dt = timed(target_seconds * 0.8)
    one_thread = None
    try:
        from threadpoolctl import threadpool_limits

        limit = threadpool_limits(limits=1, user_api="blas")
    except Exception:
        limit = None
    if limit is not None:
        with limit if hasattr(limit, "__enter__") else contextlib.nullcontext():
            one_thread, p1, reps1, dt1 = timed(target_seconds * 0.2)
    result = {
        "value": value,
        "unit": "timesteps*seqs/s",
        "cores": blas_threads,
        "cores_source": source,
        "kind": "port",
        "sample": "%s shape in fp32, one direction, first T=%i of %i frames (B=%i, n=%i), %i passes, %.1f s; "
        "per frame one SGEMM on %i BLAS threads, pointwise loop on 1 thread, as the reference's CPU path; the frame loop "
        "itself is Python (one numpy matmul and one ctypes call per frame)"
        % (name, p.T, full_T, p.B, p.n, reps, dt, blas_threads),
    }
    if one_thread is not None:
        result["value_1thread"] = one_thread
        result["sample_1thread"] = "the same with the BLAS limited to 1 thread: first T=%i frames, %i passes, %.1f s" % (p1.T, reps1, dt1)
    return result


def torch_stack_baseline(prob, dev, steps, warmup):
    """
    The same encoder forward through PyTorch's own LSTM (MIOpen on ROCm) on the same GPU: the route the reference's
    torch backend takes for an LSTM layer (pack_padded_sequence -> torch.lstm -> pad_packed_sequence,
    returnn/torch/frontend/_backend.py:2795-2822), here in its most favourable form, one bidirectional multi-layer call.
    Random weights of the same shapes (timing only).  ``packed``: the lengths are honoured, as the reference needs them;
    ``padded``: lengths ignored (not the same function, but the fastest the library can go on this shape).
    """
    import torch

    T, B, n, L, d_in = prob.T, prob.B, prob.n, prob.num_layers, prob.in_dim
    lens_cpu = torch.from_numpy(prob.lens).to(torch.int64)
    out = {"what": "torch.nn.LSTM(num_layers=%i, bidirectional=True), same shapes, same GPU; ms per forward" % L}
    for dtype in (torch.bfloat16, torch.float16):
        name = str(dtype).replace("torch.", "")
        try:
            net = torch.nn.LSTM(d_in, n, num_layers=L, bidirectional=True).to(dev).to(dtype).eval()
            x = torch.from_numpy(prob.features).to(dev).to(dtype)

            def run_packed():
                packed = torch.nn.utils.rnn.pack_padded_sequence(x, lens_cpu, enforce_sorted=False)
                return torch.nn.utils.rnn.pad_packed_sequence(net(packed)[0], total_length=T)[0]

            def run_padded():
                return net(x)[0]

            for kind, run in (("packed", run_packed), ("padded", run_padded)):
                with torch.no_grad():
                    for _ in range(max(warmup, 1)):
                        y = run()
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    for _ in range(steps):
                        y = run()
                    torch.cuda.synchronize()
                    out["%s_%s_ms" % (kind, name)] = (time.perf_counter() - t0) * 1e3 / steps
                assert tuple(y.shape) == (T, B, 2 * n)
            del net, x, y
        except Exception as exc:  # a dtype the library does not take
            out["error_%s" % name] = "%s: %s" % (type(exc).__name__, str(exc)[:200])
    return out


def bench_encoder_training(args, dev):
    """
    Config 4 with gradients: forward of the encoder, a weighted-sum loss, backward to the input and to all parameters
    (per layer and direction the gradient op, the projection's two GEMMs).  One step = forward + backward; value counts
    the op-level units of the forward pass, 12 * T * B per step.  The same step through torch.nn.LSTM beside it.
    """
    import torch

    from returnn_amd import lstm as rlstm
    from returnn_amd import synthetic

    prob = synthetic.make_encoder_config("cfg4")
    T, B, n, L = prob.T, prob.B, prob.n, prob.num_layers
    bf = torch.bfloat16
    x = torch.from_numpy(prob.features).to(dev).to(bf)
    lens = torch.from_numpy(prob.lens).to(dev)
    weight = torch.randn((T, B, 2 * n), device=dev, generator=torch.Generator(device=dev).manual_seed(0)).to(bf)

    def timed(step_fn, steps, warmup):
        for _ in range(warmup):
            step_fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step_fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    enc = rlstm.BlstmEncoder.from_params(prob.layers, device=dev, dtype=bf).train()
    params = [p for p in enc.parameters()]
    xg = x.clone().requires_grad_(True)

    def step_ours():
        for p in params:
            p.grad = None
        xg.grad = None
        y = enc(xg, seq_lens=lens)
        (y * weight).sum().backward()

    step_ms = timed(step_ours, args.steps, args.warmup)
    assert all(p.grad is not None and bool(torch.isfinite(p.grad.float()).all()) for p in params) and xg.grad is not None
    del enc, params

    torch_stack = None
    if not args.no_torch_baseline:
        lens_cpu = torch.from_numpy(prob.lens).to(torch.int64)
        torch_stack = {"what": "torch.nn.LSTM(num_layers=%i, bidirectional=True) on the packed batch, forward + backward, same GPU; ms per step" % L}
        for dtype in (torch.bfloat16, torch.float16):
            name = str(dtype).replace("torch.", "")
            try:
                net = torch.nn.LSTM(prob.in_dim, n, num_layers=L, bidirectional=True).to(dev).to(dtype).train()
                xt = x.to(dtype).clone().requires_grad_(True)
                wt = weight.to(dtype)

                def step_torch():
                    net.zero_grad(set_to_none=True)
                    xt.grad = None
                    packed = torch.nn.utils.rnn.pack_padded_sequence(xt, lens_cpu, enforce_sorted=False)
                    y = torch.nn.utils.rnn.pad_packed_sequence(net(packed)[0], total_length=T)[0]
                    (y * wt).sum().backward()

                torch_stack["packed_%s_ms" % name] = timed(step_torch, max(2, args.steps // 4), 1)
                del net, xt, wt
            except Exception as exc:
                torch_stack["error_%s" % name] = "%s: %s" % (type(exc).__name__, str(exc)[:200])

    units = 2 * L * T * B
    rec_flops = 3 * 2 * L * 8.0 * T * B * n * n  # forward GEMM, backward GEMM, weight gradient
    proj_flops = 3 * 2 * sum(2.0 * T * B * (prob.in_dim if li == 0 else 2 * n) * 4 * n for li in range(L))
    return {
        "metric": "LSTM fwd+bwd timesteps*seqs/sec (T*B/s) at n=%i" % n,
        "value": units * 1e3 / step_ms,
        "unit": "timesteps*seqs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": step_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "cfg4 training step: %i-layer bidirectional LSTM encoder forward + backward (input and all parameters), "
            "T=%i B=%i in=%i n=%i bf16, ragged=True" % (L, T, B, prob.in_dim, n),
            "calls_per_step": 4 * L,
            "units_per_step": units,
            "torch_lstm_same_gpu": torch_stack,
        },
        "roofline": {
            "bound": "mfma",
            "achieved": (rec_flops + proj_flops) / (step_ms * 1e-3) / 1e12,
            "peak": PEAK_MFMA["bf16"] / 1e12,
            "unit": "TFLOP/s",
            "frac": (rec_flops + proj_flops) / (step_ms * 1e-3) / PEAK_MFMA["bf16"],
            "traffic": None,
            "kernel": "whole step: recurrent %.3g TFLOP + projections %.3g TFLOP (forward, backward, weight gradients)"
            % (rec_flops / 1e12, proj_flops / 1e12),
        },
    }


def bench_encoder(args, dev):
    """
    Config 4: forward of the 6-layer bidirectional encoder (per layer one projection GEMM and one op call per
    direction, outputs concatenated).  One step = one forward of the stack; value counts the op-level units,
    12 * T * B per step.  The projection GEMMs (hipBLASLt) are timed again on their own to split the step time.
    """
    import torch

    from returnn_amd import lstm as rlstm
    from returnn_amd import synthetic

    prob = synthetic.make_encoder_config("cfg4")
    T, B, n, L = prob.T, prob.B, prob.n, prob.num_layers
    bf = torch.bfloat16
    enc = rlstm.BlstmEncoder.from_params(prob.layers, device=dev, dtype=bf)
    x = torch.from_numpy(prob.features).to(dev).to(bf)
    lens = torch.from_numpy(prob.lens).to(dev)
    with torch.no_grad():
        for _ in range(args.warmup):
            y = enc(x, seq_lens=lens)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            y = enc(x, seq_lens=lens)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        assert bool(torch.isfinite(y.float()).all())
        # the projections alone, same shapes and weights: one GEMM per layer into [T*B, 8n], both directions' gates
        ws = [(enc.layers[li].weights(bf), enc.in_dim if li == 0 else 2 * n) for li in range(L)]
        srcs = {d: torch.randn((T * B, d), device=dev).to(bf) for d in {enc.in_dim, 2 * n}}
        for w, d_in in ws:
            torch.addmm(w.bias, srcs[d_in], w.ff)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            for w, d_in in ws:
                torch.addmm(w.bias, srcs[d_in], w.ff)
        torch.cuda.synchronize()
        proj = time.perf_counter() - t1
    step_ms = elapsed * 1e3 / args.steps
    proj_ms = proj * 1e3 / args.steps
    del enc, y, srcs, ws
    torch_stack = None if args.no_torch_baseline else torch_stack_baseline(prob, dev, max(2, args.steps // 4), 1)
    rec_flops = 2 * L * 8.0 * T * B * n * n
    proj_flops = 2 * sum(2.0 * T * B * (prob.in_dim if li == 0 else 2 * n) * 4 * n for li in range(L))
    units = 2 * L * T * B
    return {
        "metric": "LSTM fwd timesteps*seqs/sec (T*B/s) at n=%i" % n,
        "value": units * args.steps / elapsed,
        "unit": "timesteps*seqs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": step_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "cfg4: %i-layer bidirectional LSTM encoder forward, T=%i B=%i in=%i n=%i bf16, ragged=True; "
            "per layer one projection GEMM into [T*B, 8n] and the two NativeLstm2 calls of the directions in one launch, reading "
            "their columns of it and writing their columns of one [T, B, 2n] output" % (L, T, B, prob.in_dim, n),
            "calls_per_step": 2 * L,
            "units_per_step": units,
            "projection_ms_per_step": proj_ms,
            "recurrent_and_glue_ms_per_step": step_ms - proj_ms,
            "torch_lstm_same_gpu": torch_stack,
        },
        "roofline": {
            "bound": "mfma",
            "achieved": (rec_flops + proj_flops) / (step_ms * 1e-3) / 1e12,
            "peak": PEAK_MFMA["bf16"] / 1e12,
            "unit": "TFLOP/s",
            "frac": (rec_flops + proj_flops) / (step_ms * 1e-3) / PEAK_MFMA["bf16"],
            "traffic": None,
            "kernel": "whole stack: recurrent %.3g TFLOP + projections %.3g TFLOP per step over the step time"
            % (rec_flops / 1e12, proj_flops / 1e12),
        },
    }


def cpu_baseline_gradient(name: str, target_seconds: float = 15.0):
    """Times the CPU restatement of the gradient op in its BLAS-structured form on a bounded sample."""
    import numpy

    from oracle import lstm2_oracle
    from returnn_amd import synthetic

    try:
        from threadpoolctl import threadpool_info

        blas_threads = max([int(i.get("num_threads", 1)) for i in threadpool_info() if i.get("user_api") == "blas"] or [1])
    except Exception:
        blas_threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    full_T = synthetic.make_config.__globals__["_SPECS"][name]["T"]
    T = min(full_T, 25)
    rng = numpy.random.default_rng(1)
    reps = 1
    for attempt in range(2):
        p = synthetic.make_config(name, T=T)
        Y, C, H, d, _ = lstm2_oracle.native_lstm2_fwd_blas(p.X, p.W, p.y0, p.c0, p.i)
        DY = rng.standard_normal(Y.shape, dtype=numpy.float32)
        Dd = rng.standard_normal(d.shape, dtype=numpy.float32)
        lstm2_oracle.native_lstm2_bwd_blas(p.W, p.y0, p.c0, p.i, 0, 1, Y, C, H, DY, Dd)  # warm-up (BLAS thread pool, page-in)
        t0 = time.perf_counter()
        for _ in range(reps):
            lstm2_oracle.native_lstm2_bwd_blas(p.W, p.y0, p.c0, p.i, 0, 1, Y, C, H, DY, Dd)
        dt = time.perf_counter() - t0
        if attempt == 0:
            per_frame = dt / T
            T = int(max(T, min(full_T, target_seconds / max(per_frame, 1e-9))))
            reps = int(max(1, min(50, round(target_seconds / max(per_frame * T, 1e-9)))))
    return {
        "value": reps * p.T * p.B / dt,
        "unit": "timesteps*seqs/s",
        "cores": blas_threads,
        "kind": "port",
        "sample": "gradient op, %s shape in fp32, one direction, first T=%i of %i frames (B=%i, n=%i), %i passes, %.1f s; per frame the "
        "sequential pointwise loop on 1 thread and one SGEMM on %i BLAS threads, one large SGEMM for the weight gradient, "
        "as the reference's CPU path" % (name, p.T, full_T, p.B, p.n, reps, dt, blas_threads),
    }


def bench_gradient(args, dev, cabi):
    """
    The gradient op of the workload on the results of a forward run, all resident in HBM: one direction
    (``rtn_native_lstm2_bwd``), for cfg3 both directions of the layer (``rtn_native_lstm2_bwd_multi``, or two single
    calls with ``--pair separate``).  One step = the gradient of the whole workload; value = units * K / elapsed.
    Algorithmic work per timestep x sequence:
    8 n^2 flops for the recurrent GEMM (Dy0 += DX[t] W^T) plus 8 n^2 for the weight gradient (Y^T DX).
    """
    import torch

    from returnn_amd import lib, native_op, synthetic, torch_native_op

    p = synthetic.make_config(args.workload)
    T, B, n = p.T, p.B, p.n
    dtype = p.dtype
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    dt_code = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    op = torch_native_op.make_op(native_op.NativeLstm2)
    X = torch.from_numpy(p.X).to(dev).to(act)
    W = torch.from_numpy(p.W).to(dev).to(act)
    y0 = torch.from_numpy(p.y0).to(dev).to(act)
    c0 = torch.from_numpy(p.c0).to(dev)
    msk = torch.from_numpy(p.i).to(dev)
    # cfg3 is a bidirectional layer: both directions' gradient calls in one entry unless --pair separate
    steps_of = [1, -1] if args.workload == "cfg3" else [1]
    fused = len(steps_of) > 1 and args.pair == "fused"
    fw = [op(X, W, y0, c0, msk, 0, st) for st in steps_of]
    del X
    gen = torch.Generator(device=dev).manual_seed(0)
    DY = [torch.randn(fw[0][0].shape, device=dev, generator=gen).to(act) for _ in steps_of]
    Dd = [torch.randn(fw[0][3].shape, device=dev, generator=gen) for _ in steps_of]
    DX = [torch.empty((T, B, 4 * n), dtype=act, device=dev) for _ in steps_of]
    DW = [torch.empty((n, 4 * n), dtype=torch.float32, device=dev) for _ in steps_of]
    Dy0 = [torch.empty((B, n), dtype=act, device=dev) for _ in steps_of]
    Dc0 = [torch.empty((B, n), dtype=torch.float32, device=dev) for _ in steps_of]
    each = max(cabi.rtn_native_lstm2_bwd_workspace_bytes(T, B, n, dt_code), 256)
    ws = torch.empty((each * len(steps_of),), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev)
    arr = (lib.Lstm2BwdCall * len(steps_of))()
    for k, st in enumerate(steps_of):
        Y, C, H, _ = fw[k]
        arr[k] = lib.Lstm2BwdCall(
            W.data_ptr(), y0.data_ptr(), c0.data_ptr(), msk.data_ptr(), 0, st, Y.data_ptr(), C.data_ptr(), H.data_ptr(),
            DY[k].data_ptr(), Dd[k].data_ptr(), DX[k].data_ptr(), DW[k].data_ptr(), Dy0[k].data_ptr(), Dc0[k].data_ptr())  # fmt: skip

    def call():
        if fused:
            lib.check(cabi.rtn_native_lstm2_bwd_multi(arr, len(steps_of), T, B, n, dt_code, ws.data_ptr(), ws.numel(), stream.cuda_stream))
        else:
            for k in range(len(steps_of)):
                a = arr[k]
                lib.check(cabi.rtn_native_lstm2_bwd(
                    a.W, a.y0, a.c0, a.i, a.start, a.step, a.Y, a.C, a.H, a.DY, a.Dd, a.DX, a.DW, a.Dy0, a.Dc0, T, B, n, dt_code,
                    ws.data_ptr() + k * each, each, stream.cuda_stream))  # fmt: skip

    copy_calibration(args, dev)
    for _ in range(args.warmup):
        call()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        call()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    for k in range(len(steps_of)):
        lib.check(cabi.rtn_native_lstm2_fwd_status(ws.data_ptr() + k * each, stream.cuda_stream))
        assert bool(torch.isfinite(DW[k]).all()) and bool(torch.isfinite(Dc0[k]).all())
    call_ms = elapsed * 1e3 / args.steps
    units = T * B * len(steps_of)
    flops = 16.0 * n * n * units
    peak = PEAK_MFMA[dtype]
    bwd_traffic, bwd_traffic_source = measured_traffic(
        args.workload + " gradient", 1 if (fused or len(steps_of) == 1) else len(steps_of),
        "persistent kernel, %i problem(s) per launch" % (len(steps_of) if fused else 1))
    result = {
        "metric": "LSTM gradient op timesteps*seqs/sec (T*B/s) at n=%i" % n,
        "value": units * args.steps / elapsed,
        "unit": "timesteps*seqs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": call_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": {
            "workload": "%s: NativeLstm2 gradient op, %s, T=%i B=%i n=%i %s, ragged=%s"
            % (args.workload, ("both directions, " + ("one entry" if fused else "two entries")) if len(steps_of) > 1 else "one direction",
               T, B, n, dtype, p.lens is not None),
            "calls_per_step": len(steps_of),
            "units_per_step": units,
            "plan": lib.bwd_plan_text(),
        },
        "roofline": {
            "bound": "mfma",
            "achieved": flops / (call_ms * 1e-3) / 1e12,
            "peak": peak / 1e12,
            "unit": "TFLOP/s",
            "frac": flops / (call_ms * 1e-3) / peak,
            "traffic": bwd_traffic,
            "traffic_source": bwd_traffic_source,
            "traffic_unit": "bytes per launch of the persistent kernel (transcribed from the profile summary named in traffic_source, "
            "not measured by this run); algorithmic (read H, DY, C, mask; write DX): %i"
            % (((9 * (2 if dtype == "bf16" else 4) + 4) * n + 4) * units),
            "kernel": "whole gradient call: the persistent k_lstm2_bwd_regw (or one k_bwd_step launch per frame) with the "
            "recurrent GEMM, 8*n^2 flops per unit, then the weight-gradient GEMM in rocBLAS, 8*n^2 flops per unit",
            "launch_ms": call_ms,
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_gradient(args.workload, args.cpu_seconds)
    return result


def cpu_baseline_sibling(name: str, op: str, n_in: int, target_seconds: float = 15.0):
    """Times the CPU restatement of a sibling op (plain loops, one thread) on the first frames of the workload."""
    import numpy

    from oracle import lstm2_oracle
    from returnn_amd import synthetic

    full_T = synthetic.make_config.__globals__["_SPECS"][name]["T"]
    T = 2
    rng = numpy.random.default_rng(2)
    for attempt in range(2):
        p = synthetic.make_config(name, T=T)
        if op == "generic_base":
            run = lambda: lstm2_oracle.lstm_generic_base_fwd(p.X, p.W, p.c0, p.i)  # noqa: E731
        else:
            Xr = rng.standard_normal((p.T, p.B, n_in), dtype=numpy.float32)
            Ws = numpy.concatenate([rng.standard_normal((n_in, 4 * p.n), dtype=numpy.float32) * 0.02, p.W], axis=0)
            b = numpy.zeros((4 * p.n,), numpy.float32)
            run = lambda: lstm2_oracle.lstm_low_mem_fwd(Xr, Ws, b, p.y0, p.c0, p.i, 0, 1)  # noqa: E731
        t0 = time.perf_counter()
        run()
        dt = time.perf_counter() - t0
        if attempt == 0:
            T = int(max(T, min(full_T, target_seconds / max(dt / T, 1e-9))))
    return {
        "value": p.T * p.B / dt,
        "unit": "timesteps*seqs/s",
        "cores": 1,
        "kind": "port",
        "sample": "%s forward, %s shape in fp32, first T=%i of %i frames (B=%i, n=%i%s), one pass, %.1f s, plain C loops on one thread"
        % (op, name, p.T, full_T, p.B, p.n, ", n_in=%i" % n_in if op == "low_mem" else "", dt),
    }


def bench_sibling(args, dev, cabi):
    """
    Forward pass of a sibling op on the workload's shape, inputs resident in HBM.  ``generic_base``: LstmGenericBase on the
    workload's gate inputs (8 n^2 flops per timestep x sequence).  ``low_mem``: LstmLowMem on raw input of width n_in = n
    with the stacked weight matrix (8 n^2 recurrent + 8 n_in n projection flops per unit).
    """
    import torch

    from returnn_amd import lib, synthetic

    p = synthetic.make_config(args.workload)
    T, B, n = p.T, p.B, p.n
    n_in = n
    dtype = p.dtype
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    dt_code = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    mode = lib.MODES[args.mode]
    W = torch.from_numpy(p.W).to(dev).to(act)
    y0 = torch.from_numpy(p.y0).to(dev).to(act)
    c0 = torch.from_numpy(p.c0).to(dev)
    msk = torch.from_numpy(p.i).to(dev)
    Y = torch.empty((T, B, n), dtype=act, device=dev)
    d = torch.empty((B, n), dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev)
    if args.op == "generic_base":
        Z = torch.from_numpy(p.X).to(dev).to(act)
        H = torch.empty((T, B, 4 * n), dtype=act, device=dev)
        ws = torch.empty((max(cabi.rtn_lstm_generic_base_fwd_workspace_bytes(T, B, n, dt_code, mode), 256),), dtype=torch.uint8, device=dev)
        flops = 8.0 * n * n * T * B

        def call():
            lib.check(cabi.rtn_lstm_generic_base_fwd(
                Z.data_ptr(), W.data_ptr(), c0.data_ptr(), msk.data_ptr(), Y.data_ptr(), H.data_ptr(), d.data_ptr(), T, B, n, dt_code, mode,
                ws.data_ptr(), ws.numel(), stream.cuda_stream))  # fmt: skip

        what = "LstmGenericBase forward"
    else:
        gen = torch.Generator(device=dev).manual_seed(0)
        Xr = torch.randn((T, B, n_in), device=dev, generator=gen).to(act)
        Wff = (torch.randn((n_in, 4 * n), device=dev, generator=gen) * 0.02).to(act)
        Ws = torch.cat([Wff, W], dim=0).contiguous()
        b = torch.zeros((4 * n,), dtype=act, device=dev)
        C = torch.empty((T, B, n), dtype=torch.float32, device=dev)
        ws = torch.empty((max(cabi.rtn_lstm_low_mem_fwd_workspace_bytes(T, B, n_in, n, dt_code, mode), 256),), dtype=torch.uint8, device=dev)
        flops = (8.0 * n * n + 8.0 * n_in * n) * T * B

        def call():
            lib.check(cabi.rtn_lstm_low_mem_fwd(
                Xr.data_ptr(), Ws.data_ptr(), b.data_ptr(), y0.data_ptr(), c0.data_ptr(), msk.data_ptr(), 0, 1, Y.data_ptr(), C.data_ptr(),
                d.data_ptr(), T, B, n_in, n, dt_code, mode, ws.data_ptr(), ws.numel(), stream.cuda_stream))  # fmt: skip

        what = "LstmLowMem forward, n_in=%i" % n_in
    for _ in range(args.warmup):
        call()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        call()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.check(cabi.rtn_native_lstm2_fwd_status(ws.data_ptr(), stream.cuda_stream))
    assert bool(torch.isfinite(Y.float()).all()) and bool(torch.isfinite(d).all())
    call_ms = elapsed * 1e3 / args.steps
    peak = PEAK_MFMA[dtype]
    result = {
        "metric": "%s timesteps*seqs/sec (T*B/s) at n=%i" % (what.split(",")[0], n),
        "value": T * B * args.steps / elapsed,
        "unit": "timesteps*seqs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": call_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": {
            "workload": "%s: %s, T=%i B=%i n=%i %s, ragged=%s" % (args.workload, what, T, B, n, dtype, p.lens is not None),
            "calls_per_step": 1,
            "units_per_step": T * B,
            "mode": args.mode,
        },
        "roofline": {
            "bound": "mfma",
            "achieved": flops / (call_ms * 1e-3) / 1e12,
            "peak": peak / 1e12,
            "unit": "TFLOP/s",
            "frac": flops / (call_ms * 1e-3) / peak,
            "traffic": None,
            "kernel": "whole call: the NativeLstm2 forward kernel with the sibling op's switches"
            + ("" if args.op == "generic_base" else ", after the rocBLAS projection GEMM and the bias kernel"),
            "launch_ms": call_ms,
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_sibling(args.workload, args.op, n_in, args.cpu_seconds)
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="cfg3", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "wide"])
    ap.add_argument("--mode", default="auto", choices=["auto", "persistent", "graph", "stepwise"])
    ap.add_argument("--pair", default="fused", choices=["fused", "separate"],
                    help="cfg3: issue the two directions through the multi-call entry (one launch when the device "
                         "holds both; default) or as two separate op calls")
    ap.add_argument("--op", default="fwd", choices=["fwd", "bwd", "generic_base", "low_mem"],
                    help="fwd: the forward op (default, the headline metric); bwd: the gradient op of one direction of "
                         "the workload (cfg1/cfg2/cfg3/cfg5; with cfg4: the encoder's training step, forward + backward); generic_base, low_mem: forward of the sibling ops on the workload's shape")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-step-budget", action="store_true",
                    help="skip the extra launches with the exchange waits switched off (profile runs: a kernel trace then "
                    "holds launches of the op's kernel as the op runs it, and nothing else under its name)")
    ap.add_argument("--no-torch-baseline", action="store_true", help="cfg4: skip timing the same stack through torch.nn.LSTM")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--copy-calibration-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (a kernel of known traffic, to scale "
                         "rocprofv3's FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the recurrence is one sequential chain per batch row; "
              "more GPUs would each take a share of the batch with no exchange); --gpus %i is not supported."
              % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch

    from returnn_amd import build as rbuild
    from returnn_amd import lib, synthetic

    if not os.path.exists(rbuild.LIB_PATH):
        rbuild.build_library()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    cabi = lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.workload == "cfg4":
        print(json.dumps(bench_encoder_training(args, dev) if args.op == "bwd" else bench_encoder(args, dev)))
        return
    if args.op == "bwd":
        print(json.dumps(bench_gradient(args, dev, cabi)))
        return
    if args.op in ("generic_base", "low_mem"):
        print(json.dumps(bench_sibling(args, dev, cabi)))
        return

    p = synthetic.make_config(args.workload)
    T, B, n = p.T, p.B, p.n
    dtype = p.dtype
    act = torch.bfloat16 if dtype == "bf16" else torch.float32
    dt_code = lib.DTYPE_BF16 if dtype == "bf16" else lib.DTYPE_F32
    mode = lib.MODES[args.mode]
    directions = [1, -1] if args.workload == "cfg3" else [1]

    X = torch.from_numpy(p.X).to(dev).to(act)
    W = torch.from_numpy(p.W).to(dev).to(act)
    y0 = torch.from_numpy(p.y0).to(dev).to(act)
    c0 = torch.from_numpy(p.c0).to(dev)
    msk = torch.from_numpy(p.i).to(dev)
    ws_bytes = lib.workspace_bytes(T, B, n, dt_code, mode)
    outs = []
    for _ in directions:
        outs.append(
            dict(
                Y=torch.empty((T, B, n), dtype=act, device=dev),
                C=torch.empty((T, B, n), dtype=torch.float32, device=dev),
                H=torch.empty((T, B, 4 * n), dtype=act, device=dev),
                d=torch.empty((B, n), dtype=torch.float32, device=dev),
                ws=torch.empty((max(ws_bytes, 256),), dtype=torch.uint8, device=dev),
            )
        )
    stream = torch.cuda.current_stream(dev)
    fused = len(directions) == 2 and args.pair == "fused"
    if fused:
        call_list = (lib.Lstm2Call * 2)()
        for k, o in enumerate(outs):
            call_list[k] = lib.Lstm2Call(
                X.data_ptr(), W.data_ptr(), y0.data_ptr(), c0.data_ptr(), msk.data_ptr(), 0, directions[k],
                o["Y"].data_ptr(), o["C"].data_ptr(), o["H"].data_ptr(), o["d"].data_ptr(),
            )  # fmt: skip
        ws_pair = torch.empty((max(cabi.rtn_native_lstm2_fwd_multi_workspace_bytes(2, T, B, n, dt_code, mode), 256),),
                              dtype=torch.uint8, device=dev)

    def pair_call():
        lib.check(cabi.rtn_native_lstm2_fwd_multi(call_list, 2, T, B, n, dt_code, mode, ws_pair.data_ptr(),
                                                  ws_pair.numel(), stream.cuda_stream))  # fmt: skip

    def check_status():
        if os.environ.get("RTN_LSTM2_EXCHANGE") == "3":  # no-exchange timing aid: results are invalid
            return
        if fused:
            lib.check(cabi.rtn_native_lstm2_fwd_multi_status(ws_pair.data_ptr(), 2, T, B, n, dt_code, mode, stream.cuda_stream))
        else:
            for k in range(len(directions)):
                lib.check(cabi.rtn_native_lstm2_fwd_status(outs[k]["ws"].data_ptr(), stream.cuda_stream))

    def one_call(k):
        if fused:
            return pair_call()
        o = outs[k]
        rc = cabi.rtn_native_lstm2_fwd(
            X.data_ptr(), W.data_ptr(), y0.data_ptr(), c0.data_ptr(), msk.data_ptr(), 0, directions[k],
            o["Y"].data_ptr(), o["C"].data_ptr(), o["H"].data_ptr(), o["d"].data_ptr(), T, B, n, dt_code, mode,
            o["ws"].data_ptr(), o["ws"].numel(), stream.cuda_stream,
        )  # fmt: skip
        lib.check(rc)

    copy_calibration(args, dev)

    launches = 1 if fused else len(directions)  # library entries per step
    for _ in range(args.warmup):
        for k in range(launches):
            one_call(k)
    torch.cuda.synchronize()
    check_status()

    events = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        for k in range(launches):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            one_call(k)
            e1.record(stream)
            events.append((e0, e1))
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    measuring_only = os.environ.get("RTN_LSTM2_EXCHANGE") == "3"
    check_status()
    assert measuring_only or all(bool(torch.isfinite(o["d"]).all()) for o in outs)

    call_ms = sum(a.elapsed_time(b) for a, b in events) / len(events)

    # The latency of one hand-over of values between CUs (device-scope store -> load), measured live with the library's
    # probe: a lower bound of a time step of any kernel that keeps W spread over CUs.
    probe_us = None
    probe_rounds = 4000
    probe_ws = torch.empty((32768,), dtype=torch.uint8, device=dev)
    pe = []
    for _ in range(1 + 3):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        rc = cabi.rtn_handover_latency_probe(probe_ws.data_ptr(), probe_ws.numel(), probe_rounds, stream.cuda_stream)
        e1.record(stream)
        if rc != lib.RTN_OK:
            pe = []
            break
        pe.append((e0, e1))
    torch.cuda.synchronize()
    if pe and cabi.rtn_native_lstm2_fwd_status(probe_ws.data_ptr(), stream.cuda_stream) == lib.RTN_OK:
        probe_us = min(a.elapsed_time(b) for a, b in pe[1:]) * 1e3 / probe_rounds

    # The two MFMA ceilings of the plan (no exchange): one launch of each probe, T steps -- the MFMAs alone, and the MFMAs
    # with the decomposition's partial-tile round trip through LDS.
    seq_ws = torch.empty((1 << 20,), dtype=torch.uint8, device=dev)

    def time_probe(fn):
        se = []
        for _ in range(1 + 3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            rc = fn(2 if fused else 1, T, B, n, dt_code, T, seq_ws.data_ptr(), seq_ws.numel(), stream.cuda_stream)
            e1.record(stream)
            if rc != lib.RTN_OK:
                return None
            se.append((e0, e1))
        torch.cuda.synchronize()
        return min(a.elapsed_time(b) for a, b in se[1:])

    seq_ms = time_probe(cabi.rtn_mfma_sequence_probe)
    issue_ms = time_probe(cabi.rtn_mfma_issue_probe)
    issue_clock_mhz = None
    if issue_ms is not None:
        # threads 1 and 2 of every workgroup of the issue probe leave the loop's duration in shader clocks and in ticks
        # of the constant 100 MHz clock: the clock rate the matrix cores ran at
        marks = seq_ws[: 256 * 4 * 4].view(torch.float32).view(4, 256)[:, 1:3].double().cpu()
        if float(marks[:, 1].min()) > 0:
            issue_clock_mhz = float((marks[:, 0] / marks[:, 1]).mean()) * 100.0

    # What fits behind an MFMA: the issue probe again with one, two and three vector instructions behind every MFMA
    # (a measurement variant of the library's probe for this plan's tile sequence, 64 MFMAs per wavefront and step),
    # in shader clocks per MFMA as the probe's own wavefronts count them.
    issue_clocks = None
    if (issue_clock_mhz is not None and not measuring_only and not args.no_step_budget and dt_code == lib.DTYPE_BF16 and n == 1024
            and " mt=8 nt=1 " in lib.describe_multi_plan(2 if fused else 1, T, B, n, dt_code, mode)):  # fmt: skip
        def clocks_per_mfma():
            marks = seq_ws[: 256 * 4 * 4].view(torch.float32).view(4, 256)[:, 1].double().cpu()
            return float(marks.mean()) / (T * 64.0)

        issue_clocks = {"0": clocks_per_mfma()}
        try:
            for others in (1, 2, 3):
                os.environ["RTN_LSTM2_PROBE_OTHERS"] = str(others)
                lib.reload_env()
                if time_probe(cabi.rtn_mfma_issue_probe) is None:
                    issue_clocks = None
                    break
                issue_clocks[str(others)] = clocks_per_mfma()
        finally:
            del os.environ["RTN_LSTM2_PROBE_OTHERS"]
            lib.reload_env()

    # The same launch with the reads of the hidden state switched off (a timing aid of the library: no loads from the
    # exchange ring, no delay in front of them, no waiting -- the MFMAs run on zeros, the new values are still stored;
    # results are invalid and the status word says so): what a step costs when the hidden state is there for free.
    # The difference to the measured launch is what the step spends on getting it.
    nowait_ms = None
    if "mfma_regw" in lib.describe_multi_plan(2 if fused else 1, T, B, n, dt_code, mode) and not measuring_only and not args.no_step_budget:
        os.environ["RTN_LSTM2_EXCHANGE"] = "3"
        lib.reload_env()
        try:
            ne = []
            for _ in range(1 + 3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for k in range(launches):
                    one_call(k)
                e1.record(stream)
                ne.append((e0, e1))
            torch.cuda.synchronize()
            nowait_ms = min(a.elapsed_time(b) for a, b in ne[1:]) / launches
        finally:
            del os.environ["RTN_LSTM2_EXCHANGE"]
            lib.reload_env()
        for k in range(launches):  # leave valid results behind
            one_call(k)
        torch.cuda.synchronize()
        check_status()

    units_per_step = len(directions) * T * B
    value = units_per_step * args.steps / elapsed
    units_per_launch = units_per_step // launches
    flops_per_launch = 8.0 * n * n * units_per_launch
    achieved = flops_per_launch / (call_ms * 1e-3)
    peak = PEAK_MFMA[dtype]
    bytes_per_launch = algorithmic_bytes_per_unit(n, dtype) * units_per_launch
    plan = lib.describe_multi_plan(2 if fused else 1, T, B, n, dt_code, mode)
    traffic, traffic_source = measured_traffic(args.workload, launches, plan)

    result = {
        "metric": "LSTM fwd timesteps*seqs/sec (T*B/s) at n=%i" % n,
        "value": value,
        "unit": "timesteps*seqs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": elapsed * 1e3 / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": {
            "workload": "%s: NativeLstm2 forward%s, T=%i B=%i n=%i %s, ragged=%s"
            % (args.workload,
               (" bidirectional pair (two op calls, step=+1 and step=-1, %s)"
                % ("through the multi-call entry: one launch" if fused else "two entries")) if len(directions) == 2 else "",
               T, B, n, dtype, p.lens is not None),
            "calls_per_step": len(directions),
            "launches_per_step": launches,
            "units_per_step": units_per_step,
            "mode": args.mode,
            "plan": plan,
            "sync_policy": os.environ.get("RTN_LSTM2_SYNC", "default"),
        },
        "roofline": {
            "bound": "mfma",
            "achieved": achieved / 1e12,
            "peak": peak / 1e12,
            "unit": "TFLOP/s",
            "frac": achieved / peak,
            "traffic": traffic,
            "traffic_source": traffic_source,
            "traffic_unit": "bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, transcribed from the profile summary named in "
            "traffic_source, not measured by this run); algorithmic: %i" % bytes_per_launch,
            "kernel": "%s (one launch = %i op call(s) = %i units of T*B, 8*n^2 flops each)"
            % ("k_lstm2_regw" if "mfma_regw" in plan else ("k_lstm2_mfma" if "mfma_lds" in plan else "k_step_generic"),
               len(directions) // launches, units_per_launch),
            "launch_ms": call_ms,
            **ceiling_fields(probe_us, seq_ms, issue_ms, units_per_launch // T, n, dtype, T, call_ms),
            "mfma_issue_clock_mhz": issue_clock_mhz,
            "mfma_issue_clocks_per_mfma_by_instructions_behind": issue_clocks,
            "step_budget_us": step_budget(call_ms, nowait_ms, seq_ms, issue_ms, T),
            "hbm_algorithmic_GBps": bytes_per_launch / (call_ms * 1e-3) / 1e9,
            "hbm_frac": bytes_per_launch / (call_ms * 1e-3) / PEAK_HBM,
        },
    }
    if "mode=persistent" not in plan and "kernel=mfma_lds" in plan:
        # Per-step launches: W is read from memory once per step and used once, so memory bandwidth bounds the call.
        e = 2 if dtype == "bf16" else 4
        steps_bytes = T * (4 * n * n * e) + bytes_per_launch  # W every step + the op's own streams
        result["roofline"].update({
            "bound": "hbm",
            "achieved": steps_bytes / (call_ms * 1e-3) / 1e9,
            "peak": PEAK_HBM / 1e9,
            "unit": "GB/s",
            "frac": steps_bytes / (call_ms * 1e-3) / PEAK_HBM,
            "traffic": None,
            "traffic_unit": "bytes per op call; algorithmic: %i (W once per step + X, H, Y, C, mask)" % steps_bytes,
            "kernel": "k_lstm2_mfma, one launch per step replayed through a graph (one op call = %i launches)" % T,
            "mfma_TFLOPs": achieved / 1e12,
        })
        for key in ("latency_ceiling", "frac_of_latency_ceiling", "mfma_peak_us_per_step", "achievable_mfma", "frac_of_achievable_mfma",
                    "mfma_sequence_us_per_step", "mfma_issue_us_per_step", "mfma_issue_clock_mhz", "step_budget_us", "decomposition_ceiling",
                    "mfma_issue_clocks_per_mfma_by_instructions_behind",
                    "frac_of_decomposition_ceiling"):
            result["roofline"].pop(key, None)  # they describe the exchange-bound persistent kernel
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.workload, args.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
