#!/usr/bin/env python3
"""Benchmark of sliding-window 2-simplicial attention on one MI355X.

One step = one forward + backward of the raw kernel path over one batch of synthetic
input (benchmark config 3: B=4, H=8, N=8192, D=128, w1=512, w2=32, bf16; q, k1, k2, v1,
v2 ~ N(0,1)/sqrt(D), dO ~ N(0,1)), called through the autograd Function with inputs
resident in HBM.  Prints one JSON line.

Algorithmic work (attended triples P per (batch, head), P = sum_i min(i+1,w1) min(i+1,w2)):
    forward  4*D*P flop   (logit and value contraction)
    backward 14*D*P flop  (S, dP, dV1, dV2, dK1, dK2, dQ)
`value` uses 18*D*B*H*P over the fwd+bwd time.  Each kernel is also timed on its own
through the C ABI with HIP events on the launch stream; the `roofline` object is for
the kernel with the longest launch, priced with the contractions that kernel needs
for its own outputs (fwd 2: S, O; dQ/dK2 pass 3: S, dP, G; dV2 pass 2: S, T; dK1/dV1
kernel 4: S, dP, dK1, dV1; 2*D flop each per triple).  The dQ/dK2/dV2 entry point, which
launches several kernels, is also timed whole (4 contractions: what its outputs need when
S and dP are shared).
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6   # MI355X dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name: (B, H, HK, N, D, w1, w2)
    'cfg3_raw_kernel_b4_h8_n8192_d128_w512_w32': (4, 8, 8, 8192, 128, 512, 32),
    'cfg4_long_context_b1_h16_n32768_d128_w512_w32': (1, 16, 16, 32768, 128, 512, 32),
    'cfg5_layer_b8_h8_kv4_n2048_d64_w512_w32': (8, 8, 4, 2048, 64, 512, 32),
    'tiny_b1_h2_n512_d128_w512_w32': (1, 2, 2, 512, 128, 512, 32),
    'wide_heads_b2_h8_n4096_d256_w512_w32': (2, 8, 8, 4096, 256, 512, 32),
}


def attended_triples(n, w1, w2):
    return sum(min(i + 1, w1) * min(i + 1, w2) for i in range(n))


def _median_time(fn, runs):
    ts = []
    for _ in range(runs):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return statistics.median(ts), ts


def cpu_baseline(N, D, w1, w2, slices, runs=3, naive_runs=5):
    """Two CPU legs on the host cores, both the fp32 restatement of the reference algorithm
    (`kind` "port": the reference's windowed path has no CPU implementation, its dense
    `naive_two_simplicial_attend` is a dozen lines of PyTorch that the oracle restates):

    `value`: the banded oracle, forward + backward, on `slices` complete (batch, head) slices
             of the benchmarked workload; median of `runs` runs.
    `naive_config1`: the dense naive attend at benchmark config 1 (B=1, H=4, N=128, D=32, causal,
             N(0,1) inputs), forward and forward + backward through autograd; median of
             `naive_runs` runs each.  This is the reference's own CPU-runnable case.
    """
    import torch
    from oracle import reference_attend as R
    g = torch.Generator().manual_seed(2)
    q, k1, k2, v1, v2 = [(torch.randn(1, N, slices, D, generator=g) * D ** -0.5).bfloat16().float() for _ in range(5)]
    dout = torch.randn(1, N, slices, D, generator=g).bfloat16().float()
    t, ts = _median_time(lambda: R.windowed_banded_fwd_bwd(q, k1, k2, v1, v2, dout, w1, w2, chunk=64), runs)
    flops = 18 * D * slices * attended_triples(N, w1, w2)

    # config 1: dense, causal over both key axes: sum_i (i+1)^2 attended triples per (batch, head)
    b1, h1, n1, d1 = 1, 4, 128, 32
    g = torch.Generator().manual_seed(1)
    x = [torch.randn(b1, h1, n1, d1, generator=g).requires_grad_(True) for _ in range(5)]
    do1 = torch.randn(b1, h1, n1, d1, generator=g)
    trip1 = sum((i + 1) ** 2 for i in range(n1))

    def naive_fwd():
        with torch.no_grad():
            R.naive_two_simplicial_attend(x[0], (x[1], x[2]), (x[3], x[4]), causal=True)

    def naive_fwd_bwd():
        o = R.naive_two_simplicial_attend(x[0], (x[1], x[2]), (x[3], x[4]), causal=True)
        torch.autograd.grad(o, x, do1)
    naive_fwd_bwd()
    tf, tfs = _median_time(naive_fwd, naive_runs)
    tb, tbs = _median_time(naive_fwd_bwd, naive_runs)
    return {
        'value': round(flops / t / 1e12, 4), 'unit': 'TFLOP/s', 'cores': torch.get_num_threads(), 'kind': 'port',
        'tokens_per_s': round(N * slices / t, 1),
        'sample': f'{slices} of the workload\'s (batch, head) slices, all {N} rows each, D={D} w1={w1} w2={w2}, '
                  f'fp32 banded oracle fwd+bwd, median of {runs} runs ({", ".join("%.1f" % v for v in ts)} s); '
                  f'tokens_per_s counts rows of these slices; host cpu_count={os.cpu_count()}',
        'naive_config1': {
            'workload': 'cfg1_naive_b1_h4_n128_d32_causal_fp32',
            'fwd_ms': round(tf * 1e3, 3), 'fwd_bwd_ms': round(tb * 1e3, 3),
            'fwd_tokens_per_s': round(b1 * n1 / tf, 1), 'fwd_bwd_tokens_per_s': round(b1 * n1 / tb, 1),
            'fwd_gflops': round(4 * d1 * b1 * h1 * trip1 / tf / 1e9, 2),
            'fwd_bwd_gflops': round(18 * d1 * b1 * h1 * trip1 / tb / 1e9, 2),
            'runs': naive_runs,
            'note': 'dense naive attend (what the reference tests against), autograd backward; flop counted over the '
                    'causally attended triples only, as for the GPU figures',
        },
    }


# the sources that the kernels of head dimensions 32, 64 and 128 are built from (the kernels whose HBM traffic is stored)
MEASURED_KERNEL_SOURCES = ('sa2_common.hpp', 'sa2_lds.hpp', 'sa2_fwd.hpp', 'sa2_bwd.hpp', 'sa2_bwd_q.hpp', 'sa2_bwd_kv8.hpp')


def source_digest():
    """sha256 over the sources of the measured kernels: ties a stored counter measurement to the code it was taken on."""
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, 'simplicial_attention_amd', 'csrc')
    for name in MEASURED_KERNEL_SOURCES:
        h.update(name.encode())
        h.update(open(os.path.join(csrc, name), 'rb').read())
    return h.hexdigest()[:16]


TRAFFIC_FILE = os.path.join(ROOT, 'profiles', 'hbm_traffic.json')
# the one MFMA kernel behind each single-kernel bench entry (substring of the kernel symbol)
ENTRY_KERNEL = {'fwd': 'fwd', 'bwd_dq_dk2_pass': 'bwd_q_kernel', 'bwd_dkv1': 'bwd_kv8_kernel'}


def kernel_symbol(entry, D, w2):
    if D == 256:
        return {'fwd': 'sa2::fwd_wide_kernel<256>', 'bwd_dq_dk2_pass': 'sa2::bwd_wide_q_kernel<256>', 'bwd_dkv1': 'sa2::bwd_wide_kv_kernel<256>'}.get(entry)
    if entry == 'fwd':
        return 'sa2::fwd_kernel<%d>' % D
    if entry == 'bwd_dq_dk2_pass':
        return 'sa2::bwd_q_kernel<%d, true>' % D
    if entry == 'bwd_dkv1':
        # (the entry point sa2_bwd_dkv1 has no workspace and always runs one workgroup per key slab: PARTS = false)
        return 'sa2::bwd_kv8_kernel<%d, %d, false>' % (D, 3 if D == 128 else 2)
    return None


def stored_traffic(workload, entry):
    """HBM bytes per launch of `entry` at `workload`, from the tracked counter summary (written by
    `--traffic-from`); None with a note if there is none or it was taken on other kernel sources."""
    try:
        rec = json.load(open(TRAFFIC_FILE))
    except (OSError, ValueError):
        return None, 'no profiles/hbm_traffic.json'
    e = rec.get('workloads', {}).get(workload, {}).get(entry)
    if e is None:
        return None, 'no counter run stored for this entry and workload'
    if rec.get('source_digest') != source_digest():
        return None, 'stored counter run (%s bytes) was taken on other kernel sources: rerun the --pmc passes' % e['total_bytes']
    return e['total_bytes'], 'rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a 1 GiB copy; profiles/hbm_traffic.json'


def traffic_from(directory):
    """Reads the counter CSVs of the rocprofv3 --pmc passes under `directory` (sub-directories
    <entry>_FETCH_SIZE, <entry>_WRITE_SIZE for entry in copy and the kernels; each pass is
    `rocprofv3 --pmc <counter> -d <directory>/<entry>_<counter> -o out --output-format csv --
    python3 bench.py --only <entry> [--workload W] --kernel-iters 2 --cpu-slices 0`) and writes
    profiles/hbm_traffic.json."""
    import csv
    import glob

    def per_dispatch(sub, counter, kernel_part):
        vals = []
        for f in glob.glob(os.path.join(directory, sub, '**', '*counter_collection.csv'), recursive=True):
            for row in csv.DictReader(open(f)):
                name = row.get('Kernel_Name', '')
                if kernel_part == 'fwd' and 'fwd_kernel' not in name:
                    continue
                if row.get('Counter_Name') == counter and kernel_part in name:
                    vals.append(float(row['Counter_Value']))
        return statistics.mean(vals) if vals else None
    cf = per_dispatch('copy_FETCH_SIZE', 'FETCH_SIZE', 'copyBuffer')
    cw = per_dispatch('copy_WRITE_SIZE', 'WRITE_SIZE', 'copyBuffer')
    if not cf or not cw:
        sys.exit('traffic_from: the copy calibration passes are missing under ' + directory)
    kib = float(1 << 20)                     # the copy moves 1 GiB each way
    f_fetch, f_write = kib / cf, kib / cw
    rec = {'source_digest': source_digest(), 'calibration': {'copy_FETCH_SIZE': cf, 'copy_WRITE_SIZE': cw,
                                                             'fetch_factor': round(f_fetch, 4), 'write_factor': round(f_write, 4)},
           'workloads': {}}
    for sub in sorted(os.listdir(directory)):
        if not sub.endswith('_FETCH_SIZE') or sub.startswith('copy_'):
            continue
        tag = sub[:-len('_FETCH_SIZE')]                  # <workload>__<entry>
        workload, entry = tag.split('__')
        kern = ENTRY_KERNEL.get(entry)
        if kern is None:
            continue
        fs = per_dispatch(sub, 'FETCH_SIZE', kern)
        wsz = per_dispatch(tag + '_WRITE_SIZE', 'WRITE_SIZE', kern)
        if fs is None or wsz is None:
            continue
        rd, wr = fs * f_fetch * 1024, wsz * f_write * 1024
        rec['workloads'].setdefault(workload, {})[entry] = {'read_bytes': int(rd), 'written_bytes': int(wr), 'total_bytes': int(rd + wr)}
    json.dump(rec, open(TRAFFIC_FILE, 'w'), indent=1, sort_keys=True)
    print(json.dumps(rec))

def mfma_mix_rates(iters=2048, workgroups=1024):
    """What the chip sustains on an instruction mix (profiling build of the library, sa2_prof_mix.hpp): a loop of
    independent bf16 MFMAs, two waves per SIMD, with 0 / 4+1+1 / 7+1+2 (VALU + exponential + 1 KiB LDS read) other
    instructions per MFMA, on random and on constant operands.  The nominal peak assumes the nominal clock, which the
    chip holds only on operands that do not toggle."""
    import ctypes
    import torch
    from simplicial_attention_amd import _native
    plib = _native.load_profiling()
    fn = plib.sa2_prof_mfma_mix
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    dev = torch.device('cuda:0')
    out = torch.empty(workgroups * 512, dtype=torch.float32, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream()
    g = torch.Generator(device='cpu').manual_seed(7)
    data = {'random': torch.randn(32768, generator=g).bfloat16().to(dev), 'constant': torch.ones(32768).bfloat16().to(dev)}
    mixes = {0: 'mfma_only', 1: 'plus_4_valu_1_exp_1_lds_read_per_mfma', 2: 'plus_7_valu_1_exp_2_lds_reads_per_mfma'}
    res = {}
    for dname, ops in data.items():
        for mix, mname in mixes.items():
            best = None
            for _ in range(3):
                a, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record(stream)
                rc = fn(ops.data_ptr(), out.data_ptr(), clocks.data_ptr(), mix, workgroups, iters, stream.cuda_stream)
                b_.record(stream)
                torch.cuda.synchronize()
                if rc != 0:
                    raise RuntimeError(plib.sa2_last_error().decode())
                ms = a.elapsed_time(b_)
                best = ms if best is None or ms < best else best
            c = clocks.cpu()
            tf = workgroups * 8 * iters * 16 * 32768 / (best * 1e-3) / 1e12
            res['%s_operands__%s' % (dname, mname)] = {'tflops': round(tf, 1), 'frac_of_nominal_peak': round(tf / PEAK_BF16_TFLOPS, 4),
                                                        'shader_clock_mhz': round(100.0 * int(c[0]) / max(int(c[1]), 1), 0)}
    return res


def vendor_gemm_rates(n=8192, iters=10):
    """The same question put to the vendor's GEMM: torch.matmul of two n x n bf16 matrices (hipBLASLt) on random,
    all-zero and all-one operands.  Operands that do not toggle run faster on the same code."""
    import torch
    dev = torch.device('cuda:0')
    g = torch.Generator(device='cpu').manual_seed(11)
    res = {}
    for name in ('random', 'zeros', 'ones'):
        if name == 'random':
            a, b_ = (torch.randn(n, n, generator=g).bfloat16().to(dev) for _ in range(2))
        else:
            a, b_ = (torch.full((n, n), 0.0 if name == 'zeros' else 1.0, dtype=torch.bfloat16, device=dev) for _ in range(2))
        for _ in range(3):
            torch.matmul(a, b_)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            torch.matmul(a, b_)
        torch.cuda.synchronize()
        t = (time.perf_counter() - t0) / iters
        tf = 2 * n ** 3 / t / 1e12
        res['%s_operands' % name] = {'ms': round(t * 1e3, 3), 'tflops': round(tf, 1), 'frac_of_nominal_peak': round(tf / PEAK_BF16_TFLOPS, 4)}
    return res


def vendor_attention_rates(B=4, H=8, N=8192, D=128, iters=5):
    """A third calibration point: torch's scaled_dot_product_attention (the vendor's fused attention kernels) on random
    bf16 inputs at config 3's batch, heads, length and head dimension, causal, forward and forward + backward.
    Flop: 4 N^2 D B H / 2 forward, 2.5 times that for the backward."""
    import torch
    import torch.nn.functional as F
    dev = torch.device('cuda:0')
    g = torch.Generator(device='cpu').manual_seed(5)
    q, k, v = ((torch.randn(B, H, N, D, generator=g) * D ** -0.25).bfloat16().to(dev).requires_grad_(True) for _ in range(3))
    do = torch.randn(B, H, N, D, generator=g).bfloat16().to(dev)
    fwd_flop = 4 * N * N * D * B * H / 2

    def timed(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / iters

    with torch.no_grad():
        t_f = timed(lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True))
    t_fb = timed(lambda: torch.autograd.grad(F.scaled_dot_product_attention(q, k, v, is_causal=True), (q, k, v), do))
    res = {'fwd': {'ms': round(t_f * 1e3, 3), 'tflops': round(fwd_flop / t_f / 1e12, 1)},
           'fwd_bwd': {'ms': round(t_fb * 1e3, 3), 'tflops': round(3.5 * fwd_flop / t_fb / 1e12, 1)}}
    for r in res.values():
        r['frac_of_nominal_peak'] = round(r['tflops'] / PEAK_BF16_TFLOPS, 4)
    return res


def time_raw_workload(name, steps=5, warmup=2):
    """forward + backward of the raw kernel path at workload `name` through the autograd Function: ms per step,
    TFLOP/s on the 18*D*B*H*P count and the fraction of the bf16 MFMA peak."""
    import torch
    from simplicial_attention_amd import sliding_two_simplicial_attn
    B, H, HK, N, D, w1, w2 = WORKLOADS[name]
    dev = torch.device('cuda:0')
    g = torch.Generator(device='cpu').manual_seed(3)
    mk = lambda h, sc: (torch.randn(B, N, h, D, generator=g) * sc).bfloat16().to(dev)
    ins = [mk(H, D ** -0.5)] + [mk(HK, D ** -0.5) for _ in range(4)]
    dout = mk(H, 1.0)
    ins = [t.requires_grad_(True) for t in ins]

    def step():
        out = sliding_two_simplicial_attn(ins[0], (ins[1], ins[2]), (ins[3], ins[4]), w1=w1, w2=w2, causal=True)
        return torch.autograd.grad(out, ins, dout)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / steps
    flops = 18 * D * B * H * attended_triples(N, w1, w2)
    del ins, dout
    torch.cuda.empty_cache()
    return {'ms_per_step': round(t * 1e3, 3), 'tflops': round(flops / t / 1e12, 2),
            'frac_of_bf16_peak': round(flops / t / 1e12 / PEAK_BF16_TFLOPS, 4), 'tokens_per_s': round(B * N / t, 1), 'steps': steps}


def time_train_cfg5(steps=5, warmup=2):
    """benchmark config 5: one training step (forward, loss, backward, Adam) of the byte-level LM: depth 12, dim 512,
    8 heads of 64 (4 key/value heads), every 2nd layer simplicial (w1=512, w2=32), batch 8 x 2048 random bytes; and the
    share of the six simplicial attention cores (the same Function at the layer's shape, timed alone)."""
    import torch
    from simplicial_attention_amd import sliding_two_simplicial_attn
    from simplicial_attention_amd.two_simplicial_transformer import TwoSimplicialLM
    dev = torch.device('cuda:0')
    torch.manual_seed(4)
    lm = TwoSimplicialLM(num_tokens=256, dim=512, depth=12, max_seq_len=2048, dim_head=64, heads=8,
                         two_simplicial_attn_every=2, transformer_kwargs=dict(key_value_heads=4)).bfloat16().to(dev)
    opt = torch.optim.Adam(lm.parameters(), lr=1e-4)
    tokens = torch.randint(0, 256, (8, 2049), device=dev)

    def train_step():
        opt.zero_grad(set_to_none=True)
        loss = lm(tokens, return_loss=True)
        loss.backward()
        opt.step()
        return loss
    for _ in range(max(2, warmup)):
        train_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = train_step()
    torch.cuda.synchronize()
    step_ms = (time.perf_counter() - t0) / steps * 1e3
    mk5 = lambda h: (torch.randn(8, 2048, h, 64, device=dev) * 0.125).bfloat16().requires_grad_(True)
    q5, k15, k25, v15, v25 = mk5(8), mk5(4), mk5(4), mk5(4), mk5(4)
    do5 = torch.randn(8, 2048, 8, 64, device=dev).bfloat16()

    def core():
        o = sliding_two_simplicial_attn(q5, (k15, k25), (v15, v25), w1=512, w2=32)
        torch.autograd.grad(o, (q5, k15, k25, v15, v25), do5)
    for _ in range(3):
        core()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(10):
        core()
    torch.cuda.synchronize()
    core_ms = (time.perf_counter() - t0) / 10 * 1e3
    res = {'workload': 'cfg5_training_step_depth12_dim512_b8_n2048', 'ms_per_step': round(step_ms, 3),
           'tokens_per_s': round(8 * 2048 / step_ms * 1e3, 1), 'loss': round(loss.item(), 4),
           'simplicial_core_fwd_bwd_ms_per_layer': round(core_ms, 3),
           'simplicial_cores_share_of_step': round(6 * core_ms / step_ms, 3), 'steps': steps}
    del lm, opt
    torch.cuda.empty_cache()
    return res


def time_module_cfg2(iters=50):
    """benchmark config 2: the multi-head module, tokens (2, 1024, 512), dim_head 64, 8 heads, forward, with and
    without the fused split + RMSNorm kernel; and that kernel alone at the config-3 token count."""
    import torch
    from simplicial_attention_amd import SlidingWindowTwoSimplicialMHA
    from simplicial_attention_amd.qkv_norm import FusedQKVNorm
    dev = torch.device('cuda:0')
    torch.manual_seed(1)
    m = SlidingWindowTwoSimplicialMHA(512, dim_head=64, heads=8, w1=512, w2=32).bfloat16().to(dev)
    tokens = torch.randn(2, 1024, 512, device=dev).bfloat16()

    def timed(fn, n):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        a, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        b_.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b_) / n
    res = {}
    with torch.no_grad():
        for fused in (True, False):
            m.fused_qkv_norm = fused
            res['module_fwd_ms_fused' if fused else 'module_fwd_ms_unfused'] = round(timed(lambda: m(tokens), iters), 4)
        bq, nq, hq, dq_ = 4, 8192, 8, 128
        qkv = torch.randn(bq, nq, 5 * hq * dq_, device=dev).bfloat16()
        w = torch.ones(dq_, device=dev).bfloat16()
        ms = timed(lambda: FusedQKVNorm.apply(qkv, w, w, w, w, w, hq, hq, dq_, 1e-6), 20)
        nbytes = 2 * qkv.numel() * 2 + 4 * bq * nq * 5 * hq
        res['qkv_norm_fwd'] = {'tokens': bq * nq, 'channels': 5 * hq * dq_, 'ms': round(ms, 4),
                               'hbm_bytes': nbytes, 'achieved_gbs': round(nbytes / ms / 1e6, 1), 'peak_gbs': PEAK_HBM_GBS}
    res['tokens_per_s'] = round(2 * 1024 / res['module_fwd_ms_fused'] * 1e3, 1)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=10)
    ap.add_argument('--warmup', type=int, default=3)
    ap.add_argument('--workload', default='cfg3_raw_kernel_b4_h8_n8192_d128_w512_w32', choices=sorted(WORKLOADS))
    ap.add_argument('--cpu-slices', type=int, default=4, help='(batch, head) slices of the CPU baseline sample (0 = skip)')
    ap.add_argument('--kernel-iters', type=int, default=5, help='launches per kernel for the per-kernel timing')
    ap.add_argument('--no-other-workloads', dest='other_workloads', action='store_false',
                    help='skip the other benchmark workloads (config 4, the config-5 layer and training step, the config-2 module) that the default run times after config 3')
    ap.add_argument('--traffic-from', default=None, metavar='DIR', help='no GPU work: read the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE passes under DIR and write profiles/hbm_traffic.json')
    ap.add_argument('--only', default=None, help='time only this entry through the C ABI (fwd, bwd_delta, bwd_dq_dkv2, bwd_dkv1, bwd_dq_dk2_pass), `mfma_mix`: the MFMA rates this chip sustains on three instruction mixes with random and constant operands; `copy`: a 1 GiB device copy that calibrates HBM counters; `module_cfg2`: the module forward of config 2 and the fused qkv-norm kernel; `train_cfg5`: one training step of the config-5 language model; for profiling')
    args = ap.parse_args()
    if args.traffic_from:
        traffic_from(args.traffic_from)
        return
    if args.gpus != 1:
        print('bench.py: this build runs on one GPU; --gpus must be 1 (no multi-GPU path exists)', file=sys.stderr)
        sys.exit(2)

    import torch
    from simplicial_attention_amd import _native, sliding_two_simplicial_attn
    if not torch.cuda.is_available():
        print('bench.py: no GPU visible', file=sys.stderr)
        sys.exit(1)
    if not os.path.exists(_native.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    lib = _native.load()

    B, H, HK, N, D, w1, w2 = WORKLOADS[args.workload]
    dev = torch.device('cuda:0')
    if args.only == 'train_cfg5':
        print(json.dumps(time_train_cfg5(args.steps, args.warmup)))
        return
    if args.only == 'module_cfg2':
        print(json.dumps(time_module_cfg2()))
        return
    if args.only == 'mfma_mix':
        print(json.dumps({'instruction_mix_loop': mfma_mix_rates(), 'torch_matmul_bf16_8192': vendor_gemm_rates(),
                          'torch_sdpa_causal_b4_h8_n8192_d128': vendor_attention_rates()}))
        return
    if args.only == 'copy':
        # plain device copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(args.kernel_iters):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({'copy_bytes_read': 1 << 30, 'copy_bytes_written': 1 << 30, 'launches': args.kernel_iters}))
        return
    g = torch.Generator(device='cpu').manual_seed(2)
    mk = lambda h, s: (torch.randn(B, N, h, D, generator=g) * s).bfloat16().to(dev)
    q = mk(H, D ** -0.5)
    k1, k2, v1, v2 = (mk(HK, D ** -0.5) for _ in range(4))
    dout = mk(H, 1.0)
    ins = [t.requires_grad_(True) for t in (q, k1, k2, v1, v2)]

    def fwd():
        return sliding_two_simplicial_attn(ins[0], (ins[1], ins[2]), (ins[3], ins[4]), w1=w1, w2=w2, causal=True)

    def step():
        out = fwd()
        return torch.autograd.grad(out, ins, dout)

    step_s = fwd_s = float('nan')
    if args.only is None:
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        step_s = (time.perf_counter() - t0) / args.steps

    # forward only (same API, no graph kept)
    if args.only is None:
        with torch.no_grad():
            for _ in range(2):
                fwd()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(max(3, args.steps)):
                fwd()
            torch.cuda.synchronize()
            fwd_s = (time.perf_counter() - t0) / max(3, args.steps)

    # ---- per-kernel timing through the C ABI, HIP events on the launch stream
    P = attended_triples(N, w1, w2)
    unit = 2 * D * B * H * P   # one contraction over all triples
    stream = torch.cuda.current_stream()
    sh = stream.cuda_stream
    arg = _native.tensor_arg
    prob = _native.problem(B, N, H, HK, D, w1, w2, True, D ** -0.5)
    qd, k1d, k2d, v1d, v2d = (t.detach() for t in ins)
    out = torch.empty_like(qd)
    res = torch.empty_like(qd)
    lse = torch.empty(B, H, N, dtype=torch.float32, device=dev)
    delta = torch.empty_like(lse)
    dq = torch.empty_like(qd)
    dk1, dk2, dv1, dv2 = (torch.empty_like(k1d) for _ in range(4))
    five = (arg(qd), arg(k1d), arg(k2d), arg(v1d), arg(v2d))
    ws_bytes = lib.sa2_bwd_workspace_bytes(prob)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    # the forward's per-offset value partials, as the autograd Function keeps them
    saved = t_save = m_save = None
    from simplicial_attention_amd.two_simplicial_attention import save_partials_max_bytes
    if 0 < lib.sa2_saved_t_bytes(prob) <= save_partials_max_bytes():      # (0: this head dimension keeps no partials)
        t_save = torch.empty(lib.sa2_saved_t_bytes(prob), dtype=torch.uint8, device=dev)
        m_save = torch.empty(lib.sa2_saved_m_bytes(prob), dtype=torch.uint8, device=dev)
        saved = _native.saved_arg(t_save, m_save)
    launches = {
        'fwd': (2, lambda: lib.sa2_fwd(prob, *five, arg(out), arg(res), lse.data_ptr(), saved, sh)),
        'bwd_delta': (0, lambda: lib.sa2_bwd_delta(prob, arg(out), arg(res), arg(dout), delta.data_ptr(), sh)),
        'bwd_dq_dkv2': (4, lambda: lib.sa2_bwd_dq_dkv2(prob, *five, arg(dout), lse.data_ptr(), delta.data_ptr(), saved, arg(dq), arg(dk2),
                                                      arg(dv2), ws.data_ptr(), ws_bytes, sh)),
        'bwd_dkv1': (4, lambda: lib.sa2_bwd_dkv1(prob, *five, arg(dout), lse.data_ptr(), delta.data_ptr(), arg(dk1), arg(dv1), sh)),
    }
    # the MFMA kernel of the dQ/dK2/dV2 entry point alone: the profiling build of the library launches only
    # that kernel when SA2_BWD_PASS=first is set (the product library has no such switch)
    plib = _native.load_profiling()

    def dq_dk2_kernel_alone():
        os.environ['SA2_BWD_PASS'] = 'first'
        try:
            return plib.sa2_bwd_dq_dkv2(prob, *five, arg(dout), lse.data_ptr(), delta.data_ptr(), saved, arg(dq),
                                        arg(dk2), arg(dv2), ws.data_ptr(), ws_bytes, sh)
        finally:
            del os.environ['SA2_BWD_PASS']
    launches['bwd_dq_dk2_pass'] = (3, dq_dk2_kernel_alone)
    kernels = {}
    if args.only is not None:
        # the later kernels read what the earlier ones wrote: run the chain once, untimed
        for name in ('fwd', 'bwd_delta'):
            if name == args.only:
                break
            _native.check(launches[name][1]())
        launches = {args.only: launches[args.only]}
    for name, (ncontr, fn) in launches.items():
        _native.check(fn())
        torch.cuda.synchronize()
        evs = []
        for _ in range(args.kernel_iters):
            a, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            _native.check(fn())
            b_.record(stream)
            evs.append((a, b_))
        torch.cuda.synchronize()
        ms = statistics.mean(a.elapsed_time(b_) for a, b_ in evs)
        kernels[name] = {'ms': round(ms, 4), 'contractions': ncontr,
                         'tflops': round(ncontr * unit / (ms * 1e-3) / 1e12, 2) if ncontr else None}
    if args.only is not None:
        print(json.dumps({'workload': args.workload, 'kernels': kernels}))
        return
    hbm_bytes = {'fwd': 7 * B * N * H * D * 2 + 4 * B * H * N, 'bwd_delta': 3 * B * N * H * D * 2 + 4 * B * H * N}
    # entries that are exactly one kernel launch (the dQ/dK2/dV2 entry point launches several: its MFMA kernel is
    # timed alone as bwd_dq_dk2_pass)
    multi = ('bwd_dq_dkv2',)
    single = [k for k in kernels if kernels[k]['contractions'] and k not in multi]
    dom = max(single, key=lambda k: kernels[k]['ms'])
    achieved = kernels[dom]['tflops']
    traffic, traffic_note = stored_traffic(args.workload, dom)
    # the dominant kernel inside the step: the whole backward through sa2_bwd (HIP events on the launch stream) minus
    # the stand-alone times of its other entries
    in_step_ms = None
    if dom == 'bwd_dkv1':
        g5 = [torch.empty_like(qd)] + [torch.empty_like(k1d) for _ in range(4)]
        bwd_all = lambda: lib.sa2_bwd(prob, *five, arg(out), arg(res), arg(dout), lse.data_ptr(), saved, delta.data_ptr(),
                                      arg(g5[0]), arg(g5[1]), arg(g5[2]), arg(g5[3]), arg(g5[4]), ws.data_ptr(), ws_bytes, sh)
        _native.check(bwd_all())
        torch.cuda.synchronize()
        evs = []
        for _ in range(args.kernel_iters):
            a, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            _native.check(bwd_all())
            b_.record(stream)
            evs.append((a, b_))
        torch.cuda.synchronize()
        bwd_ms = statistics.mean(a.elapsed_time(b_) for a, b_ in evs)
        kernels['bwd_whole'] = {'ms': round(bwd_ms, 4), 'contractions': 7, 'tflops': round(7 * unit / (bwd_ms * 1e-3) / 1e12, 2)}
        in_step_ms = round(bwd_ms - kernels['bwd_delta']['ms'] - kernels['bwd_dq_dkv2']['ms'], 4)
    roofline = {'bound': 'mfma', 'kernel': dom, 'kernel_symbol': kernel_symbol(dom, D, w2), 'achieved': achieved, 'peak': PEAK_BF16_TFLOPS, 'unit': 'TFLOP/s',
                'frac': round(achieved / PEAK_BF16_TFLOPS, 4), 'traffic': traffic, 'traffic_note': traffic_note,
                'launch_ms': kernels[dom]['ms'],
                'in_step_ms': in_step_ms,
                'frac_in_step': round(kernels[dom]['contractions'] * unit / (in_step_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4) if in_step_ms else None,
                'in_step_note': 'launch_ms: the kernel alone in a loop; in_step_ms: the whole backward (sa2_bwd) minus its other entries timed alone',
                'flops_per_launch': kernels[dom]['contractions'] * unit}

    total_flops = 9 * unit          # 18*D*B*H*P
    value = total_flops / step_s / 1e12
    result = {
        'metric': 'fwd+bwd TFLOP/s, bf16 2-simplicial attn N=%d w1=%d w2=%d' % (N, w1, w2),
        'value': round(value, 2), 'unit': 'TFLOP/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': round(step_s * 1e3, 3), 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'bf16', 'data': 'synthetic',
        'config': {'workload': args.workload, 'batch': B, 'heads': H, 'kv_heads': HK, 'seq_len': N, 'dim_head': D,
                   'w1': w1, 'w2': w2},
        'frac_of_bf16_peak': round(value / PEAK_BF16_TFLOPS, 4),
        'tokens_per_s': round(B * N / step_s, 1),
        'fwd': {'ms': round(fwd_s * 1e3, 3), 'tflops': round(2 * unit / fwd_s / 1e12, 2),
                'frac_of_bf16_peak': round(2 * unit / fwd_s / 1e12 / PEAK_BF16_TFLOPS, 4),
                'tokens_per_s': round(B * N / fwd_s, 1),
                'hbm_gbs_algorithmic': round(hbm_bytes['fwd'] / (kernels['fwd']['ms'] * 1e-3) / 1e9, 1)},
        'kernels': kernels,
        'roofline': roofline,
    }
    # what the MFMA pipe sustains on this chip, measured in the same run: the nominal peak holds for operands that do
    # not toggle; on random operands the clock drops under the power limit
    sustained = mfma_mix_rates(iters=1024)
    roofline['sustained_on_this_chip'] = sustained
    rnd = sustained['random_operands__mfma_only']['tflops']
    roofline['frac_of_sustained_random_operand_mfma_rate'] = round(achieved / rnd, 4)
    result['frac_of_sustained_random_operand_mfma_rate'] = round(value / rnd, 4)
    if args.other_workloads and args.workload == 'cfg3_raw_kernel_b4_h8_n8192_d128_w512_w32':
        # the other benchmark workloads, timed in the same run (each at least 5 steps)
        torch.cuda.empty_cache()
        other = {}
        for name in ('cfg4_long_context_b1_h16_n32768_d128_w512_w32', 'cfg5_layer_b8_h8_kv4_n2048_d64_w512_w32'):
            other[name] = time_raw_workload(name, steps=5 if 'cfg4' in name else 10)
        other['cfg5_training_step_depth12_dim512_b8_n2048'] = time_train_cfg5(steps=5)
        other['cfg2_module_forward_b2_n1024_dim512'] = time_module_cfg2(iters=20)
        result['other_workloads'] = other
    if args.cpu_slices > 0:
        result['cpu_baseline'] = cpu_baseline(N, D, w1, w2, args.cpu_slices)
    print(json.dumps(result))


if __name__ == '__main__':
    main()
