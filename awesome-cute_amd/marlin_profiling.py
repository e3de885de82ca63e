"""Kernel-time sweep over the linear layers of LLaMA-class models, the counterpart
of the reference's gemm/marlin_gemm/marlin_profiling.py:87-121: for every layer
shape, per-channel and group-128 scales, batch 1 and 16, quantise a random
weight (gen_quant4, reference marlin_profiling.py:13-50), run marlin.mul and
write one row per case to a CSV.

Two times are reported per case.  `resident_us` launches over one weight buffer,
as the reference's loop does (marlin_profiling.py:60-70); on MI355X such a buffer
stays in the 256 MB Infinity Cache whenever it fits.  `hbm_us` rotates over
enough copies of the weights that every launch reads them from HBM.  Both are
means over `iters` launches replayed from one HIP graph, so that host time does
not count, as with the reference's torch.profiler device_time.

    python awesome-cute_amd/marlin_profiling.py --models 7B --iters 200 --out marlin_perf.csv
"""
import argparse
import csv
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import marlin  # noqa: E402

# (k, n) of the fused qkv, attention output, fused gate/up and down projections
# (reference marlin_profiling.py:88-113)
MODELS = {
    '7B': [(4096, 3 * 4096), (4096, 4096), (4096, 2 * 10752), (10752, 4096)],
    '13B': [(5120, 3 * 5120), (5120, 5120), (5120, 2 * 13568), (13568, 5120)],
    '33B': [(6656, 3 * 6656), (6656, 6656), (6656, 2 * 17664), (17664, 6656)],
    '70B': [(8192, 3 * 8192), (8192, 8192), (8192, 2 * 21760), (21760, 8192)],
}
GROUP_SIZES = (-1, 128)
BATCHES = (1, 16)

# bytes of weights to rotate over so that none survive in the Infinity Cache
_ROTATE_BYTES = 2 * 256 * 1024 * 1024


def gen_quant4(k, n, groupsize=-1, dev='cuda', seed=0):
    """Random (k, n) half weight, quantised and packed: returns the fake-quantised
    weight, the packed words (k/16, 2n) and the packed scales."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    w = torch.randn((k, n), dtype=torch.half, device=dev, generator=gen)
    ref, q, s = marlin.quantize(w, groupsize)
    del w
    B = marlin.pack_weights(q)
    del q
    return ref, B, marlin.pack_scales(s, groupsize != -1)


def _graph_us(fn, iters, stream):
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for i in range(iters):
            fn(i)
    graph.replay()
    torch.cuda.synchronize()
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    cur = torch.cuda.current_stream()
    t0.record(cur)
    graph.replay()
    t1.record(cur)
    torch.cuda.synchronize()
    return t0.elapsed_time(t1) * 1e3 / iters


def run_profiling(m, n, k, group_size=-1, iters=1000, model='', check=True, dev='cuda',
                  quantised=None):
    """One row of the sweep.  `quantised` may carry gen_quant4's result for (k, n,
    group_size) so that several batch sizes share it."""
    ref, B, s = quantised if quantised is not None else gen_quant4(k, n, group_size, dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(m)
    A = torch.randn((m, k), dtype=torch.half, device=dev, generator=gen)
    C = torch.zeros((m, n), dtype=torch.half, device=dev)
    workspace = torch.zeros(n // 128 * 16, dtype=torch.int, device=dev)
    weight_bytes = k * n // 2
    copies = max(2, min(64, -(-_ROTATE_BYTES // weight_bytes)))
    Bs = [B] + [B.clone() for _ in range(copies - 1)]

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        # the first call on a stream allocates the library's scratch buffer
        marlin.mul(A, B, C, s, workspace)
        side.synchronize()
        err = None
        if check:
            want = torch.matmul(A.float(), ref.float())
            err = ((C.float() - want).abs().max() / want.abs().max()).item()
            if not err <= 1e-2:
                raise AssertionError(f"m={m} n={n} k={k} group={group_size}: error {err:.3g}")
            if workspace.any().item():
                raise AssertionError("workspace not restored to zero")
    resident = _graph_us(lambda i: marlin.mul(A, B, C, s, workspace), iters, side)
    hbm = _graph_us(lambda i: marlin.mul(A, Bs[i % copies], C, s, workspace), iters, side)
    _, plan = marlin.plan(m, n, k, group_size)
    return {
        'shape(m_n_k_group)': f"{model}_{m}_{n}_{k}_{group_size}",
        'resident_us': f"{resident:.3f}",
        'hbm_us': f"{hbm:.3f}",
        'hbm_weight_GBps': f"{weight_bytes / hbm / 1e3:.0f}",
        'kernel': {1: 'stream', 2: 'prefill', 3: 'strips'}[plan['kernel']],
        'workgroups': plan['grid'],
        'max_rel_err': '' if err is None else f"{err:.2e}",
    }


def sweep(models, iters=1000, check=True, dev='cuda', out=None, log=print):
    rows = []
    for model in models:
        for k, n in MODELS[model]:
            for group_size in GROUP_SIZES:
                quantised = gen_quant4(k, n, group_size, dev)
                for batch in BATCHES:
                    row = run_profiling(batch, n, k, group_size, iters, model, check, dev,
                                        quantised)
                    rows.append(row)
                    log(', '.join(f"{a}={b}" for a, b in row.items()))
                del quantised
                torch.cuda.empty_cache()
    if out:
        with open(out, 'w', newline='') as f:
            wr = csv.DictWriter(f, fieldnames=list(rows[0].keys()))
            wr.writeheader()
            wr.writerows(rows)
    return rows


def main():
    ap = argparse.ArgumentParser(description=__doc__.split('\n')[0])
    ap.add_argument('--models', default=','.join(MODELS), help='comma-separated subset of ' + ','.join(MODELS))
    ap.add_argument('--iters', type=int, default=1000)
    ap.add_argument('--no-check', action='store_true', help='skip the comparison with torch.matmul')
    ap.add_argument('--out', default='marlin_perf.csv')
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit('marlin_profiling needs a GPU')
    sweep([x.strip() for x in args.models.split(',')], args.iters, not args.no_check, out=args.out,
          log=lambda line: print(line, flush=True))


if __name__ == '__main__':
    main()
