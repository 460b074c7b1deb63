"""Benchmark of the LookupFFN hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg1|cfg3|cfg3bf16|cfg3f16|cfg2b64|cmp512|cfg4|cfg5]

A step is one forward pass of the layer over one batch of synthetic tokens that
is already resident in HBM: fused LayerNorm+projection+hash kernel -> gather-add
kernel (+bias), i.e. LookupFFN.forward in eval mode.  Prints ONE JSON line:

  value        whole-layer forward tokens/s (BASELINE.json's metric, config 2 by default)
  roofline     the gather-add kernel against the bound that binds it.  The table-major
               kernels serve every row read from LDS, so the bound is the LDS read
               path: achieved = B*T*Do*e row bytes per launch / the kernel's average
               duration (HIP events on the launch stream, inside the timed region),
               peak = 256 B/clk/CU x 256 CUs x 2.4 GHz.  Beside it: the compulsory
               HBM bytes (tables + codes + scores + output, each once) and the
               fabric traffic measured with rocprofv3 --pmc, as fractions of 8 TB/s,
               and the "logical" rate (every row read counted as memory traffic)
               as logical_gbps.  Small shapes run the token-major form (rows from
               L2): there the bound is "hbm" and achieved counts the compulsory bytes.
               16-bit rows (cfg3bf16, cfg3f16) halve the LDS bytes and are bound by the
               vector ALU instead (bound "valu": widenings + multiply-adds per second
               against 256 CUs x 4 SIMDs x 16 lanes x 2.4 GHz), the LDS rate beside it.
  cpu_baseline the CPU oracle (OpenMP C restatement of the reference's layer) on a
               bounded sample of the same workload, on the host cores of this box

One GPU only: this path has no multi-GPU form in this build.
"""
from __future__ import annotations

import argparse
import statistics
import json
import math
import os
import sys
import time
from argparse import Namespace

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

WORKLOADS = {
    # name: (B, H, T, S, Do, table dtype)          BASELINE.json configs[0..2]
    "cfg1": dict(B=256, H=256, T=32, S=256, Do=256, bf16=False,
                 desc="config 1: 2x128 tokens, d=256, 32 tables x 256 x 256 fp32"),
    "cfg2": dict(B=16384, H=768, T=128, S=256, Do=768, bf16=False,
                 desc="config 2 (RoBERTa-base): 32x512 tokens, d=768 padded to 1024, 128 tables x 256 x 768 fp32"),
    "cfg3": dict(B=16384, H=1024, T=512, S=256, Do=1024, bf16=False,
                 desc="config 3: 16384 tokens, d=1024, 512 tables x 256 x 1024 fp32"),
    "cfg3bf16": dict(B=16384, H=1024, T=512, S=256, Do=1024, bf16=True,
                     desc="config 3: 16384 tokens, d=1024, 512 tables x 256 x 1024 bf16 rows, fp32 accumulate"),
    # config 3 with half rows: the row format of the reference's own reduced-precision gather
    # (PL/gather/cuda/extension/gather_kernel_fp16.cu), fp32 accumulate here
    "cfg3f16": dict(B=16384, H=1024, T=512, S=256, Do=1024, bf16=False, f16=True,
                    desc="config 3: 16384 tokens, d=1024, 512 tables x 256 x 1024 half (fp16) rows, fp32 accumulate"),
    # config 2 with the 64 x 64 block-diagonal BH4 the reference's training configs use
    # (cfgs/roberta/small-512/lookup-t128-s8-bh4.py:25-26) instead of the sign diagonal
    "cfg2b64": dict(B=16384, H=768, T=128, S=256, Do=768, bf16=False, bs=64,
                    desc="config 2 shape with BH4 block size 64 (the reference's training config): 32x512 tokens, "
                         "d=768 padded to 1024, 4 stages of 16 blocks 64x64, 128 tables x 256 x 768 fp32"),
    # the shape of the reference's own timing script (PL/compare.py:11-22: 64 x 512 tokens, hidden 512,
    # 128 tables x 256, BH4 block size 64, output 512), which it runs beside a dense FFN 512 -> 2048 -> 512
    "cmp512": dict(B=32768, H=512, T=128, S=256, Do=512, bf16=False, bs=64,
                   desc="the reference's compare.py shape: 64x512 tokens, d=512, BH4 block size 64 (2 repeats x 4 stages "
                        "of 8 blocks), 128 tables x 256 x 512 fp32"),
    # BASELINE.json configs[3]: the 12-layer encoder with every FFN a config-2 LookupFFN
    "cfg4": dict(B=16384, H=768, T=128, S=256, Do=768, bf16=False,
                 desc="config 4: 12-layer pre-norm RoBERTa-base encoder (hidden 768, 12 heads, seq 512, batch 32), "
                      "every FFN a config-2 LookupFFN"),
    # BASELINE.json configs[4]: the backward at the config-2 shape, codes drawn Zipf(1.1)
    "cfg5": dict(B=16384, H=768, T=128, S=256, Do=768, bf16=False,
                 desc="config 5: backward at the config-2 shape, codes Zipf(s=1.1) over 256 entries"),
}

# LDS read path of CDNA4: 256 bytes per clock per CU; 256 CUs at the 2.4 GHz peak engine clock.
# (A read-only probe on this part reaches 180 B/clk/CU with linear ds_read_b128 from 16 wavefronts
# per CU and 145 B/clk/CU with 16 lanes per randomly chosen 256-byte row, the gather's pattern.)
LDS_READ_PEAK_GBS = 256 * 256 * 2.4
LDS_PROBED_GBS = 145 * 256 * 2.4          # what that probe reads for the gather's access pattern
LDS_PEAK_BASIS = ("256 B/clk/CU x 256 CUs x 2.4 GHz; a read-only ds_read_b128 probe on this part reaches 180 B/clk/CU "
                  "(linear) and 145 B/clk/CU (16 lanes per random 256-byte row, this kernel's pattern)")
# Vector ALU: 4 SIMDs x 16 lanes per CU, one fp32 operation per lane and clock (packed fp32 instructions are
# switched off in this build), 256 CUs at 2.4 GHz
VALU_PEAK_GOPS = 256 * 4 * 16 * 2.4
# L2 read path: 16 channels x 128 B/clk per XCD, 8 XCDs, 2.4 GHz
L2_READ_PEAK_GBS = 16 * 128 * 8 * 2.4
# HBM-side bytes per launch of the gather (cfg5: scatter) kernels measured with rocprofv3 --pmc
# (FETCH_SIZE + WRITE_SIZE, scaled by a copy kernel of known size), and the kernel form they were
# measured on; the summaries are kept under profiles/.  Reported only while the library still runs
# that form for the workload (a figure for another kernel would be stale).
MEASURED_TRAFFIC = {
    "cfg2": {"bytes": 253060326, "form": "record stream (four lanes per token), 1648 tokens per workgroup"},
    "cfg2b64": {"bytes": 253056190, "form": "record stream (four lanes per token), 1648 tokens per workgroup"},
    "cfg3": {"bytes": 1072501827, "form": "record stream (four lanes per token), 2048 tokens per workgroup"},
    "cfg3bf16": {"bytes": 757701017, "form": "record stream (four lanes per token), 1024 tokens per workgroup"},
    "cfg3f16": {"bytes": 770419298, "form": "record stream (four lanes per token), 1024 tokens per workgroup"},
    "cfg5": {"bytes": 942744083, "form": "sorted"},
}


def measured_traffic(workload, form):
    rec = MEASURED_TRAFFIC.get(workload)
    return rec["bytes"] if rec and rec["form"] == form else None


def row_format(wl):
    """The C ABI's row_format of a workload's tables: 0 fp32, 1 bfloat16, 2 half."""
    return 1 if wl["bf16"] else (2 if wl.get("f16") else 0)


def gather_form(B, T, S, Do, fmt):
    """Which gather kernel the layer runs for a shape and row format, as a short string (host-side queries only)."""
    import ctypes

    from lookupffn_amd import _lib
    lib = _lib.load()
    tok, stride, nbytes = ctypes.c_int32(0), ctypes.c_int64(0), ctypes.c_int64(0)
    _lib.check(lib.lffn_lookup_gather_records_plan_rows(B, T, S, Do, fmt, ctypes.byref(tok), ctypes.byref(stride),
                                                        ctypes.byref(nbytes)), "records plan")
    if nbytes.value > 0:
        return f"record stream (four lanes per token), {tok.value} tokens per workgroup"
    ws = ctypes.c_int64(0)
    _lib.check(lib.lffn_lookup_gather_workspace_bytes(B, T, S, Do, fmt, ctypes.byref(ws)), "workspace query")
    form = ctypes.c_int32(-1)
    tokens = lib.lffn_lookup_gather_ws_plan(B, T, S, Do, fmt, ws.value, ctypes.byref(form))
    if form.value == 4:
        return "table split"
    if form.value == 3:
        return f"record stream (four lanes per token), {tokens} tokens per workgroup"
    return "token-major" if form.value == 0 else f"{form.value} table(s) per LDS buffer, {tokens} tokens per workgroup"


def build_layer(wl, device):
    import torch

    import lookupffn_amd

    cfg = Namespace(hidden_size=wl["H"], ffn_num_table=wl["T"], ffn_table_size=wl["S"],
                    layer_norm_eps=1e-5, projection_type="bh4", block_size=wl.get("bs", 1))
    g = torch.Generator().manual_seed(1234)
    layer = lookupffn_amd.LookupFFN(cfg, wl["Do"]).eval()
    p = layer.hash.projection
    with torch.no_grad():
        if p.block_size == 1:
            # seeded +-1 sign diagonals, scaled by 1/sqrt(D) so that each of the four
            # (diagonal, Hadamard) stages is orthonormal
            sign = 2.0 * torch.randint(0, 2, p.weight.shape, generator=g).float() - 1.0
            p.weight.copy_(sign / math.sqrt(p.padded_in_dim))
        else:
            # the reference's initialisation, PL/lookup.py:22-23
            p.weight.copy_(torch.randn(p.weight.shape, generator=g) / math.sqrt(p.block_size * p.padded_in_dim))
        layer.tables.copy_(0.02 * torch.randn(layer.tables.shape, generator=g))
        layer.bias.copy_(0.001 * torch.randn(layer.bias.shape, generator=g))
    x = torch.randn(wl["B"], wl["H"], generator=g)
    layer = layer.to(device)
    if wl["bf16"]:
        layer.tables.data = layer.tables.data.to(torch.bfloat16)
    elif wl.get("f16"):
        layer.tables.data = layer.tables.data.to(torch.float16)
    return layer, x


def cpu_baseline(layer, x, wl, budget_s=12.0):
    """The oracle's whole-layer forward on a slice of the same tokens, all host cores."""
    import numpy as np

    import oracle

    npf = lambda t: t.detach().float().cpu().numpy()
    p = layer.hash.projection
    args = (npf(layer.LayerNorm.weight), npf(layer.LayerNorm.bias), np.float32(layer.LayerNorm.eps),
            npf(p.weight), npf(p.bias), npf(layer.tables), npf(layer.bias))
    n = min(wl["B"], 2048)
    xs = np.ascontiguousarray(npf(x)[:n])
    oracle.lookup_ffn(xs, *args, decay=np.float32(p.decay_coeff))          # warm-up (page-in)
    reps, t_total = 0, 0.0
    while reps < 3 or (t_total < budget_s and reps < 5000):
        t0 = time.perf_counter()
        oracle.lookup_ffn(xs, *args, decay=np.float32(p.decay_coeff))
        t_total += time.perf_counter() - t0
        reps += 1
    cpu_model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            cpu_model = next(l.split(":", 1)[1].strip() for l in f if l.startswith("model name"))
    except (OSError, StopIteration):
        pass
    out = {"value": n * reps / t_total, "unit": "tokens/s", "cores": oracle.num_threads(), "kind": "port",
           "cpu_model": cpu_model,
           "sample": f"first {n} of {wl['B']} tokens, full tables, {reps} passes of the OpenMP C oracle "
                     f"(whole layer, fp32{' on the 16-bit-rounded tables' if row_format(wl) else ''}), {t_total:.1f} s"}
    # the reference's own x86 kernels (compiled from its sources), gather + code/score legs only
    try:
        import torch
        ga = oracle.load_ref("gather_add_cpu")
        if ga is not None and wl["S"] == 256 and n % 64 == 0:
            torch.set_num_threads(oracle.num_threads())
            T, S = wl["T"], wl["S"]
            idx = torch.randint(0, S, (n, T), dtype=torch.int32) + torch.arange(T, dtype=torch.int32)[None] * S
            w = torch.rand(n, T)
            flat = layer.tables.detach().float().cpu().reshape(T * S, wl["Do"])
            ga.weighted_vector_gather_add_avx2_par(idx, flat, w)
            t0 = time.perf_counter()
            r = 0
            while r < 3 or time.perf_counter() - t0 < 3.0:
                ga.weighted_vector_gather_add_avx2_par(idx, flat, w)
                r += 1
            out["reference_gather_tokens_per_s"] = n * r / (time.perf_counter() - t0)
    except Exception as e:   # the reference build is optional
        out["reference_gather_error"] = repr(e)
    return out


def settle(step, cap_s=1.5, min_s=0.25, tol=0.02):
    """Untimed: run `step` in batches of about 20 ms until three batches in a row take within `tol` of the
    batch before them (the first few hundred launches after idle run at lower engine clocks), for at least
    `min_s` and at most about `cap_s` seconds.  Returns
    (steps run, milliseconds spent).  The timed region that follows is not touched."""
    import torch
    torch.cuda.synchronize()
    t_start = time.perf_counter()
    t0 = time.perf_counter()
    step()
    torch.cuda.synchronize()
    one = max(time.perf_counter() - t0, 1e-6)
    batch = max(2, min(2000, int(0.02 / one)))            # about 20 ms of work per batch
    steps, prev, quiet = 1, None, 0
    while time.perf_counter() - t_start < cap_s:
        t0 = time.perf_counter()
        for _ in range(batch):
            step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        steps += batch
        quiet = quiet + 1 if (prev is not None and abs(dt - prev) <= tol * prev) else 0
        prev = dt
        if quiet >= 2 and time.perf_counter() - t_start >= min_s:
            break
    return steps, (time.perf_counter() - t_start) * 1e3


def calibrate_copy(dev):
    """One plain 1 GiB device-to-device copy: a kernel of known traffic for scaling
    FETCH_SIZE / WRITE_SIZE in a rocprofv3 --pmc run of this command."""
    import torch
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    dst.copy_(src)                 # reads 1 GiB, writes 1 GiB
    torch.cuda.synchronize()
    del src, dst


def zipf_codes(B, T, S, gen, s=1.1):
    """Per (token, table) a rank drawn with p_r ~ r^-s, mapped to a table entry by a
    fixed seeded permutation per table."""
    import torch
    p = 1.0 / torch.arange(1, S + 1, dtype=torch.float64) ** s
    rank = torch.multinomial(p / p.sum(), B * T, replacement=True, generator=gen).reshape(B, T)
    perm = torch.stack([torch.randperm(S, generator=gen) for _ in range(T)], dim=0)      # [T, S]
    return torch.gather(perm.t().contiguous(), 0, rank).to(torch.int32)                  # perm[t][rank[b,t]]


def main_backward(args):
    """Backward of the layer's operators at the config-2 shape: gradient w.r.t. the
    scores (indexed inner product), the tables (scatter-add), and, in one kernel, z
    (closed-form score derivative), the projection input (the four diagonal x Hadamard
    stages transposed), the diagonals and the projection bias."""
    import numpy as np
    import torch

    from lookupffn_amd import _lib, ops
    _lib.load()
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    dev = torch.device("cuda:0")
    wl = WORKLOADS["cfg5"]
    B, H, T, S, Do = wl["B"], wl["H"], wl["T"], wl["S"], wl["Do"]
    layer, x_cpu = build_layer(wl, dev)
    g = torch.Generator().manual_seed(4321)
    code_cpu = zipf_codes(B, T, S, g)
    z_cpu = torch.randn(B, T, 8, generator=g)
    g_out_cpu = torch.randn(B, Do, generator=g)
    score_cpu = 1.0 - torch.rand(B, T, generator=g)
    code, z, g_out, score = code_cpu.to(dev), z_cpu.to(dev), g_out_cpu.to(dev), score_cpu.to(dev)
    z2 = z.reshape(B, T * 8).contiguous()
    tables = layer.tables.detach()
    flat = tables.reshape(T * S, Do)
    p = layer.hash.projection
    D = p.padded_in_dim
    diag = p.weight.detach().reshape(1, 4, D).contiguous()
    h = x_cpu.to(dev)                      # the projection's input (the LayerNorm output in the layer)

    def step():
        # LookupGather.backward (grad score and grad tables in one call: the score-gradient kernel and the sorted
        # scatter share one slice-major copy of the gradient) + ProjectHash.backward (grad of the projection
        # input, of the diagonals and of the projection bias), as a training step runs them
        g_score, g_tables = ops.lookup_backward(code, score, g_out, tables)
        g_h, g_diag, g_bias = ops.project_hash_bwd(h, diag, z2, g_score, float(p.decay_coeff), float(1 - p.decay_coeff))
        return g_score, g_tables, g_h, g_diag, g_bias

    if args.calibrate_copy:
        calibrate_copy(dev)
    settle_steps, settle_ms = (0, 0.0) if args.no_settle else settle(step)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step()
    torch.cuda.synchronize()
    sec = time.perf_counter() - t0
    # The roofline's kernel: the table gradient (transpose/pack, sort, sorted accumulate).  The step issues
    # both gradients in one call, which events on the stream cannot split, so its duration comes from a loop
    # of its own right after the timed one: the same launches, event pairs around each.
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in evs:
        a.record()
        ops.lookup_scatter(code, score, g_out, S)
        b.record()
    torch.cuda.synchronize()
    scatter_ms = sum(a.elapsed_time(b) for a, b in evs) / args.steps
    scatter_bytes = B * T * Do * 4 * 2 + B * T * 8 + B * Do * 4
    achieved = scatter_bytes / (scatter_ms * 1e-3) / 1e9
    row_bytes = B * T * Do * 4                                            # gradient rows read, one per (token, table)
    compulsory = T * S * Do * 4 + B * T * 8 + B * Do * 4                  # tables written, codes + scores + g read, each once

    def timed(fn, n=10):
        fn(); torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        b.record(); torch.cuda.synchronize()
        return a.elapsed_time(b) / n
    inner_ms = timed(lambda: ops.lookup_inner(code, g_out, tables))
    both_ms = timed(lambda: ops.lookup_backward(code, score, g_out, tables))
    g_score = ops.lookup_inner(code, g_out, tables)
    bwd_proj_ms = timed(lambda: ops.project_hash_bwd(h, diag, z2, g_score, 0.7, 0.3))

    res = {
        "metric": "LookupFFN bwd tokens/s + scatter-add GB/s as % of HBM peak, RoBERTa-base shape, Zipf(1.1) codes",
        "value": B * args.steps / sec, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic (seeded; codes Zipf(1.1) through a seeded permutation per table)",
        "config": {"workload": wl["desc"], "tokens": B, "tables": T, "table_size": S, "d_out": Do,
                   "step": "one call: inner product (grad score) + scatter-add (grad tables); one kernel: score "
                           "derivative, transposed BH4(block 1)x4, grad of diagonals and bias"},
        # the sorted scatter reads every (token, table)'s 3 KB gradient row from L2 into registers (the
        # gradient matrix stays in the L2s) and writes each table row once: its bound is the L2 read path
        "roofline": {"bound": "l2", "kernel": "lookup_scatter (three launches: transpose, sort + slice-major copy, sorted accumulate)",
                     "achieved": row_bytes / (scatter_ms * 1e-3) / 1e9, "peak": L2_READ_PEAK_GBS, "unit": "GB/s",
                     "frac": row_bytes / (scatter_ms * 1e-3) / 1e9 / L2_READ_PEAK_GBS,
                     "peak_basis": "16 channels x 128 B/clk per XCD x 8 XCDs x 2.4 GHz",
                     "traffic": measured_traffic("cfg5", "sorted"),
                     "row_read_bytes": row_bytes, "avg_kernel_ms": scatter_ms,
                     "hbm": {"compulsory_bytes": compulsory, "frac_of_peak": compulsory / (scatter_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
                     "logical_gbps": achieved, "algorithmic_bytes": scatter_bytes},
        "stages_ms": {"lookup_backward (both gradients, one call)": both_ms, "lookup_inner alone": inner_ms,
                      "scatter_add alone": scatter_ms, "project_hash_bwd": bwd_proj_ms},
        "settle_steps": settle_steps, "settle_ms": settle_ms,
    }
    if not args.no_cpu_baseline:
        import oracle
        n = 1024
        npf = lambda t: t.detach().float().cpu().numpy()
        idx_n = (code[:n] + torch.arange(T, device=dev, dtype=torch.int32)[None] * S).cpu().numpy().astype(np.int32)
        g_n, w_n, z_n = npf(g_out[:n]), npf(score[:n]), npf(z[:n])
        flat_n = npf(flat)
        reps, tt = 0, 0.0
        while reps < 2 or (tt < 10.0 and reps < 1000):
            t0 = time.perf_counter()
            gs = oracle.indexed_inner_product(idx_n, g_n, flat_n)
            oracle.scatter_add(idx_n, g_n, w_n, T * S)
            gz = oracle.code_score_bwd(z_n, gs)
            oracle.fht(np.ascontiguousarray(gz.reshape(n, T * 8)))
            tt += time.perf_counter() - t0
            reps += 1
        res["cpu_baseline"] = {"value": n * reps / tt, "unit": "tokens/s", "cores": oracle.num_threads(), "kind": "port",
                               "sample": f"first {n} tokens, {reps} passes of the C oracle's inner product, scatter-add "
                                         f"(serial by definition), score derivative and one FHT, {tt:.1f} s"}
    else:
        res["cpu_baseline"] = None
    print(json.dumps(res))


def main_encoder(args):
    """End-to-end forward of the 12-layer encoder (attention, LayerNorm, embeddings in
    PyTorch-ROCm; LookupFFN on this package's kernels) and the LookupFFN share of it."""
    import torch

    import lookupffn_amd
    from lookupffn_amd import _lib
    _lib.load()
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    dev = torch.device("cuda:0")
    wl = WORKLOADS["cfg4"]
    batch, seq = 32, 512
    cfg = Namespace(hidden_size=768, num_attention_heads=12, attention_head_size=64,
                    attention_probs_dropout_prob=0.1, hidden_dropout_prob=0.1, layer_norm_eps=1e-5,
                    num_hidden_layers=12, vocab_size=50265, max_position_embeddings=512, type_vocab_size=1,
                    pad_token_id=1, ffn_num_table=wl["T"], ffn_table_size=wl["S"], projection_type="bh4",
                    block_size=1)
    torch.manual_seed(1234)
    model = lookupffn_amd.Lookup(cfg).eval()
    with torch.no_grad():
        for layer in model.encoder.layer:
            p = layer.FFN.hash.projection
            p.weight.copy_((2.0 * torch.randint(0, 2, p.weight.shape).float() - 1.0) / math.sqrt(p.padded_in_dim))
    model = model.to(dev)
    ids = torch.randint(0, cfg.vocab_size, (batch, seq), device=dev)
    tt = torch.zeros_like(ids)
    pos = torch.arange(seq, device=dev)[None].expand(batch, seq).contiguous()
    mask = torch.ones(batch, seq, device=dev)

    ffn_events = []

    def pre_hook(mod, inp):
        e = torch.cuda.Event(enable_timing=True); e.record(); mod._ev0 = e

    def post_hook(mod, inp, out):
        e = torch.cuda.Event(enable_timing=True); e.record(); ffn_events.append((mod._ev0, e))

    def run():
        with torch.no_grad():
            return model(ids, tt, pos, mask)[0]

    settle_steps, settle_ms = (0, 0.0) if args.no_settle else settle(run)
    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    sec = time.perf_counter() - t0
    # LookupFFN share: a separate pass with events around every FFN call
    hooks = []
    for layer in model.encoder.layer:
        hooks.append(layer.FFN.register_forward_pre_hook(pre_hook))
        hooks.append(layer.FFN.register_forward_hook(post_hook))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        run()
    e1.record()
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    ffn_ms = sum(a.elapsed_time(b) for a, b in ffn_events) / 5
    total_ms = e0.elapsed_time(e1) / 5
    res = {
        "metric": "12-layer RoBERTa-base encoder with LookupFFN, fwd tokens/s and LookupFFN share of time",
        "value": batch * seq * args.steps / sec, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": sec / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic (random token ids, random-init weights, seeded sign diagonals)",
        "config": {"workload": wl["desc"], "tokens": batch * seq, "layers": 12, "hidden": 768, "heads": 12,
                   "seq_len": seq, "batch": batch, "tables": wl["T"], "table_size": wl["S"],
                   "attention": "torch scaled_dot_product_attention, fp32"},
        "roofline": None, "cpu_baseline": None,
        "lookupffn_ms_per_forward": ffn_ms, "forward_ms_with_events": total_ms,
        "lookupffn_share": ffn_ms / total_ms,
        "settle_steps": settle_steps, "settle_ms": settle_ms,
    }
    print(json.dumps(res))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="cfg2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph", action="store_true",
                    help="forward workloads: capture the step in a HIP graph and time replays (the launch-bound "
                         "small configurations); the gather's own duration is then measured in an eager loop")
    ap.add_argument("--two-kernels", action="store_true",
                    help="small forward workloads: keep the projection+hash kernel and the gather kernel apart "
                         "instead of the one-launch form of the layer (for comparison)")
    ap.add_argument("--no-settle", action="store_true",
                    help="skip the untimed, bounded settle loop that precedes the warm-up (profiler runs)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device-to-device copy, so that a rocprofv3 --pmc run of "
                         "this command holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the LookupFFN hot path on ONE GPU only "
              "(no multi-GPU form exists); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.workload == "cfg5":
        return main_backward(args)
    if args.workload == "cfg4":
        return main_encoder(args)

    import torch

    from lookupffn_amd import _lib, ops
    _lib.load()                       # fail here, loudly, if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    dev = torch.device("cuda:0")
    wl = WORKLOADS[args.workload]
    B, H, T, S, Do = wl["B"], wl["H"], wl["T"], wl["S"], wl["Do"]
    layer, x_cpu = build_layer(wl, dev)
    x = x_cpu.to(dev)
    fmt = row_format(wl)
    esz = 2 if fmt else 4
    gather_bytes = B * T * Do * esz + B * T * 8 + B * Do * 4

    block = layer.hash.projection.block_size != 1

    def hash_front():
        if block:        # one kernel: LayerNorm, BH4 on the matrix cores, mix + hash
            return layer.hash.forward_block(x, layer_norm=layer.LayerNorm)
        return layer.hash.forward_fused(x, layer_norm=layer.LayerNorm)

    if args.two_kernels:
        type(layer).FUSED_LAYER_MAX_TOKENS = 0
    with torch.no_grad():
        fused_layer = layer.can_fuse_layer(x)      # few tokens: the layer is one launch, gather included
    # many tokens, diagonal BH4, fp32 tables: the projection kernel writes the gather's record stream itself
    st = layer._inference_state()
    rec_plan = None
    if not fused_layer and T % 2 == 0 and st is not None:
        rec_plan = ops.lookup_gather_records_plan(B, T, S, Do, fmt)

    def records_front():
        if block:
            return ops.ln_bh4_block_hash_records_direct(x, st["ln_w"], st["ln_b"], st["eps"], layer.hash.folded_weight(),
                                                        st["pbias"], T, st["decay"], st["res_coef"], rec_plan)
        return ops.ln_project_hash_records_direct(x, st["ln_w"], st["ln_b"], st["eps"], st["diag"], st["pbias"],
                                                  T, st["decay"], st["res_coef"], rec_plan)

    def step(events=None):
        # exactly what LookupFFN.forward runs in eval mode (checked below), with an
        # event pair around the gather launch
        with torch.no_grad():
            if fused_layer:
                if events is not None:
                    events[0].record()
                out = layer._forward(x)
                if events is not None:
                    events[1].record()
                return out
            if rec_plan is not None:
                records = records_front()
                if events is not None:
                    events[0].record()
                out = ops.lookup_gather_records_direct(records, rec_plan, st["tables"], st["obias"], None, B)
                if events is not None:
                    events[1].record()
                return out
            code, score = hash_front()
            if events is not None:
                events[0].record()
            out = ops.lookup_gather(code, score, layer.tables, layer.bias)
            if events is not None:
                events[1].record()
        return out

    with torch.no_grad():
        assert torch.equal(step(), layer(x)), "bench step and LookupFFN.forward disagree"

    if args.calibrate_copy:
        calibrate_copy(dev)

    # untimed and bounded: lets the engine clocks come up before the warm-up, so that a short run
    # (--steps 20 --warmup 5) reads the same step time as a long one
    settle_steps, settle_ms = (0, 0.0) if args.no_settle else settle(step)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    if args.graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            graph_out = step()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(graph_out, step()), "graph replay and eager step disagree"
        t0 = time.perf_counter()
        for i in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        sec = time.perf_counter() - t0
        timed_evs = evs
        for i in range(args.steps):                       # the gather's duration: eager, with events
            step(evs[i])
        torch.cuda.synchronize()
    else:
        # one launch of a few microseconds per step: an event pair around every launch would be a third
        # of the step, so every eighth step carries one
        stride = 8 if fused_layer else 1
        timed_evs = evs[::stride]
        t0 = time.perf_counter()
        for i in range(args.steps):
            out = step(evs[i] if i % stride == 0 else None)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        sec = t1 - t0
    gather_ms = sum(a.elapsed_time(b) for a, b in timed_evs) / len(timed_evs)
    logical_gbps = gather_bytes / (gather_ms * 1e-3) / 1e9
    row_bytes = B * T * Do * esz                                          # one row per (token, table)
    compulsory = T * S * Do * esz + B * T * 8 + B * Do * 4                # tables, codes + scores, output: each once
    form = "whole layer in one launch (rows from L2)" if fused_layer else gather_form(B, T, S, Do, fmt)
    lds_bound = not fused_layer and form != "token-major"
    traffic = measured_traffic(args.workload, form)
    hbm = {"compulsory_bytes": compulsory, "frac_of_peak": compulsory / (gather_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
           "measured_traffic_bytes": traffic,
           "measured_frac_of_peak": None if traffic is None else traffic / (gather_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    if lds_bound and fmt != 0 and form.startswith("record stream"):
        # 16-bit rows in the four-lanes kernel: half the LDS bytes per column, and one (half: v_fma_mix_f32) or two
        # (bfloat16: widen, multiply-add) vector-ALU operations per column and (token, table): that kernel is bound
        # by vector-ALU issue, not by the LDS
        vec_ops = B * T * Do * (2 if fmt == 1 else 1)
        achieved = vec_ops / (gather_ms * 1e-3) / 1e9
        lds_rate = row_bytes / (gather_ms * 1e-3) / 1e9
        roofline = {"bound": "valu", "kernel": "lookup_gather: " + form, "achieved": achieved, "peak": VALU_PEAK_GOPS,
                    "unit": "Gop/s", "frac": achieved / VALU_PEAK_GOPS,
                    "peak_basis": "256 CUs x 4 SIMDs x 16 lanes x 2.4 GHz, one fp32 operation per lane and clock (no packed "
                                  "fp32); counted: " + ("a widening and a multiply-add" if fmt == 1 else "one v_fma_mix_f32") +
                                  " per column of every (token, table) row",
                    "traffic": traffic, "vector_ops": vec_ops, "avg_kernel_ms": gather_ms,
                    "lds": {"row_read_bytes": row_bytes, "achieved_gbps": lds_rate, "frac_of_peak": lds_rate / LDS_READ_PEAK_GBS},
                    "hbm": hbm, "logical_gbps": logical_gbps, "algorithmic_bytes": gather_bytes}
    elif lds_bound:
        achieved = row_bytes / (gather_ms * 1e-3) / 1e9
        roofline = {"bound": "lds", "kernel": "lookup_gather: " + form, "achieved": achieved, "peak": LDS_READ_PEAK_GBS,
                    "unit": "GB/s", "frac": achieved / LDS_READ_PEAK_GBS, "frac_of_probed": achieved / LDS_PROBED_GBS,
                    "peak_basis": LDS_PEAK_BASIS, "traffic": traffic,
                    "row_read_bytes": row_bytes, "avg_kernel_ms": gather_ms, "hbm": hbm,
                    "logical_gbps": logical_gbps, "algorithmic_bytes": gather_bytes}
    else:
        achieved = compulsory / (gather_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "kernel": ("lookup_ffn_fused: " if fused_layer else "lookup_gather: ") + form,
                    "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                    "traffic": traffic, "avg_kernel_ms": gather_ms, "hbm": hbm,
                    "logical_gbps": logical_gbps, "algorithmic_bytes": gather_bytes}

    # stage breakdown (outside the timed region)
    def timed(fn, n=20):
        fn(); torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        b.record(); torch.cuda.synchronize()
        return a.elapsed_time(b) / n
    def front():
        if rec_plan is not None:
            return records_front()
        return hash_front()
    with torch.no_grad():
        hash_ms = None if fused_layer else timed(front)

    # Warm and cold medians of single launches (outside the timed region).  Warm: back to
    # back, the tables still in the caches from the launch before.  Cold: a 1 GiB fill
    # between the launches pushes the tables out of the L2s and the 256 MB Infinity Cache.
    def single(fn, reps, flush=None):
        ts = []
        for _ in range(reps):
            if flush is not None:
                flush.add_(1.0)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(); fn(); b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b))
        return statistics.median(ts)
    with torch.no_grad():
        if fused_layer:
            gather_only = step
        else:
            if rec_plan is not None:
                records = front()
                gather_only = lambda: ops.lookup_gather_records_direct(records, rec_plan, st["tables"], st["obias"], None, B)
            else:
                code, score = hash_front()
                gather_only = lambda: ops.lookup_gather(code, score, layer.tables, layer.bias)
        warm_gather, warm_step = single(gather_only, 25), single(step, 25)
        flush = torch.zeros(1 << 28, dtype=torch.float32, device=dev)
        cold_gather, cold_step = single(gather_only, 15, flush), single(step, 15, flush)
        del flush

    res = {
        "metric": "LookupFFN fwd tokens/s + gather-add GB/s as % of HBM peak, RoBERTa-base",
        "value": B * args.steps / sec,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sec / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("f32", "bf16 rows, f32 accumulate", "f16 rows, f32 accumulate")[fmt],
        "data": ("synthetic (seeded N(0,1) tokens, N(0,1)/sqrt(64 D) block weights, N(0,0.02) tables)" if block else
                 "synthetic (seeded N(0,1) tokens, seeded +-1/sqrt(D) sign diagonals, N(0,0.02) tables)"),
        "config": {"workload": wl["desc"], "tokens": B, "d_model": H, "fht_dim": layer.hash.projection.padded_in_dim,
                   "tables": T, "table_size": S, "d_out": Do,
                   "step": ("one kernel: LayerNorm + BH4(block 64)x4 on fp32 MFMA + mix + hash (weights folded once, "
                            "outside the step)" + (", written as the gather's record stream" if rec_plan is not None else "") +
                            "; one kernel: gather-add + bias") if block else
                           ("one kernel: LayerNorm + BH4(block 1)x4 + mix + hash + gather-add + bias" if fused_layer else
                            ("one kernel: LayerNorm + BH4(block 1)x4 + mix + hash, written as the gather's record stream; "
                             "one kernel: gather-add + bias") if rec_plan is not None else
                            "one kernel: LayerNorm + BH4(block 1)x4 + mix + hash; one kernel: gather-add + bias")},
        "roofline": roofline,
        "stages_ms": ({"whole_layer": gather_ms} if fused_layer else
                      {("layernorm_bh4block_hash" if block else "layernorm_project_hash"): hash_ms,
                       "gather_add": gather_ms}),
        "gather_tokens_per_s": B / (gather_ms * 1e-3),
        "single_launch_median_ms": {"gather_warm": warm_gather, "gather_cold": cold_gather,
                                    "step_warm": warm_step, "step_cold": cold_step,
                                    "cold": "1 GiB fill between launches (tables evicted from L2 and Infinity Cache)"},
        "launch": "HIP graph replay" if args.graph else "eager",
        "settle_steps": settle_steps, "settle_ms": settle_ms,
    }
    if args.workload == "cmp512":
        # the dense block the reference's script times beside the layer (PL/compare.py:40-45), same tokens,
        # fp32 on the same GPU through PyTorch-ROCm
        dense = torch.nn.Sequential(torch.nn.LayerNorm(H, eps=1e-5), torch.nn.Linear(H, 4 * H), torch.nn.GELU(),
                                    torch.nn.Linear(4 * H, Do)).to(dev).eval()
        with torch.no_grad():
            res["dense_ffn_same_gpu"] = {"ms": timed(lambda: dense(x), 10), "dtype": "f32",
                                         "what": f"LayerNorm + Linear({H},{4 * H}) + GELU + Linear({4 * H},{Do}), torch"}
            res["dense_ffn_same_gpu"]["tokens_per_s"] = B / (res["dense_ffn_same_gpu"]["ms"] * 1e-3)
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(layer, x_cpu, wl)
    else:
        res["cpu_baseline"] = None
    print(json.dumps(res))


if __name__ == "__main__":
    main()
