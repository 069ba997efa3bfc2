"""Decode-throughput benchmark of the DF11 hot path on one MI355X.

A step is one decode of a Llama-3-8B-shaped decoder block (q, k, v, o, gate, up,
down; 218 103 808 BF16 elements, random-init N(0, 0.02)) compressed as ONE DF11
stream, from HBM-resident compressed inputs into one contiguous BF16 buffer.
Prints one JSON line: GB/s of algorithmic traffic (compressed bytes read + BF16
bytes written), the HBM-roofline fraction of the decode kernel, and the CPU
oracle timed on the host cores of the same machine.
"""
import argparse
import json
import os
import sys
import threading
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
LLAMA3_8B_BLOCK = [("q_proj", 4096, 4096), ("k_proj", 1024, 4096), ("v_proj", 1024, 4096),
                   ("o_proj", 4096, 4096), ("gate_proj", 14336, 4096), ("up_proj", 14336, 4096),
                   ("down_proj", 4096, 14336)]


def algorithmic_bytes(n_bytes, n_elements, n_luts):
    """Bytes a decode must move: bitstream, sign|mantissa, gaps, block positions, LUT rows in;
    BF16 out.  (The kernel reads its 512-byte-granular positions, 32 B per block, instead of
    the 4-byte block position; the extra is not counted as useful traffic.)"""
    n_blocks = -(-n_bytes // 4096)
    return n_bytes + n_elements + 320 * n_blocks + 4 * (n_blocks + 1) + 256 * n_luts + 2 * n_elements


def make_block(torch, device):
    parts = []
    for i, (_, rows, cols) in enumerate(LLAMA3_8B_BLOCK):
        g = torch.Generator(device=device).manual_seed(1000 + i)
        parts.append((torch.randn(rows * cols, generator=g, device=device) * 0.02).to(torch.bfloat16))
    return torch.cat(parts)


def cpu_baseline(stream, original_u16, budget_s=12.0):
    """Times the CPU oracle (scalar C restatement of the reference kernel) on a bounded
    run of consecutive bitstream blocks of the same stream, on the host's cores, and
    compares what it decoded with the original BF16 words."""
    from oracle import df11_oracle as O
    n_bytes = stream["encoded_exponent"].size
    n_blocks = -(-n_bytes // 4096)
    n_threads = max(1, min(16, len(os.sched_getaffinity(0)), int(os.environ.get("OMP_NUM_THREADS", "16"))))
    out = np.zeros(stream["sign_mantissa"].size, np.uint16)
    args = (stream["luts"], stream["encoded_exponent"], stream["sign_mantissa"],
            stream["output_positions"], stream["gaps"])

    def run(b0, b1):
        O.c_decode(*args, block_range=(b0, b1), out=out)

    probe = min(n_blocks, 200)
    t0 = time.perf_counter()
    run(0, probe)
    per_block_1t = (time.perf_counter() - t0) / probe
    # whole stream if it fits the budget of CPU work, else a prefix of it; repeated so
    # that about `budget_s` core-seconds are spent, and the median pass is reported
    sample = int(min(n_blocks, max(n_threads, budget_s / per_block_1t)))
    repeats = int(max(1, min(15, budget_s / (sample * per_block_1t))))
    bounds = [sample * i // n_threads for i in range(n_threads + 1)]
    times = []
    for _ in range(repeats):
        threads = [threading.Thread(target=run, args=(bounds[i], bounds[i + 1])) for i in range(n_threads)]
        t0 = time.perf_counter()
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        times.append(time.perf_counter() - t0)
    dt = float(np.median(times))
    pos = stream["output_positions"].astype(np.int64)
    elems = int(pos[min(sample, pos.size - 1)] - pos[0])
    bytes_done = sample * (4096 + 320 + 4) + 3 * elems
    single = bytes_done / (sample * per_block_1t)
    first, last = int(pos[0]), int(pos[min(sample, pos.size - 1)])
    bit_exact = bool(np.array_equal(out[first:last], original_u16[first:last]))
    return {
        "value": bytes_done / dt / 1e9, "unit": "GB/s", "cores": n_threads, "host_cores": os.cpu_count(),
        "host_cores_usable": len(os.sched_getaffinity(0)), "kind": "port",
        "bit_exact": bit_exact,
        "sample": f"first {sample} of {n_blocks} bitstream blocks of the same stream ({elems} elements), "
                  f"median of {repeats} passes of {dt:.2f} s, scalar C restatement of the reference "
                  f"kernel, one thread per core over disjoint block ranges",
        "single_thread_GBps": single / 1e9,
    }


def side_measurements(torch, dev, embedding_shape=True):
    """Kernel-time throughput of the same entry point on other inputs: the 4096x14336
    matrix (and the 151936x4096 embedding-shaped tensor) under each adversarial exponent
    distribution, and N(0, 0.02) tensors of the sizes a per-Linear compression produces.
    Every stream is held in enough device copies, decoded in turn, that no launch finds its
    input in the 256 MB memory-side cache: `hbm_frac` is HBM-fed; the figures for one copy
    decoded over and over are reported beside it as `same_copy_*`.
    Returns (mixes, sizes): name -> figures."""
    import bench_extra

    def figures(w):
        r = bench_extra.time_copies_in_turn(torch, w)
        return {"n_elements": r["n_elements"], "kernel": r["kernel"], "device_copies": r["device_copies"],
                "ms_per_launch": r["copies_in_turn_ms_per_launch"],
                "GBps": r["algorithmic_bytes"] / (r["copies_in_turn_ms_per_launch"] * 1e-3) / 1e9,
                "hbm_frac": r["copies_in_turn_hbm_frac"],
                "same_copy_ms_per_launch": r["same_copy_ms_per_launch"], "same_copy_frac": r["same_copy_hbm_frac"],
                "bit_exact": r["bit_exact"], "bits_per_exponent": r["bits_per_exponent"],
                "max_code_bits": r["max_code_bits"], "compressed_over_bf16": r["compressed_over_bf16"]}

    mixes, sizes = {}, {}
    shapes = [(4096, 14336)] + ([(151936, 4096)] if embedding_shape else [])
    for rows, cols in shapes:
        # the four distributions of the benchmark configuration, and on the matrix two more
        # whose chunks take many table lookups (sparse weights, six- and seven-bit codes)
        for kind in bench_extra.MIXES + (bench_extra.EXTRA_MIXES if (rows, cols) == (4096, 14336) else ()):
            w = bench_extra.make_mix(torch, kind, rows * cols, dev, seed=7)
            mixes[f"{kind} {rows}x{cols}"] = figures(w)
            del w
            torch.cuda.empty_cache()
    for rows, cols in ((4096, 4096), (4096, 14336)):
        g = torch.Generator(device=dev).manual_seed(0)
        w = (torch.randn(rows * cols, generator=g, device=dev) * 0.02).to(torch.bfloat16)
        sizes[f"normal {rows}x{cols}"] = figures(w)
        del w
    torch.cuda.empty_cache()
    return mixes, sizes


def end_to_end(torch, dev, num_tokens, batch_sizes=(1, 64)):
    """Generation with the Qwen3-8B-shaped model (random-init, greedy, 64 random prompt ids)
    in BF16 and with every linear and the embedding in DF11, at each batch size: tokens per
    second of both, their ratio, peak device memory, and whether logits and tokens are
    identical.  Same fields as the reference's benchmark script prints
    (reference: inference.py:62-97)."""
    from dfloat11_amd import inference
    t0 = time.perf_counter()
    out = {}
    for r in inference.compare_synthetic("qwen3-8b", list(batch_sizes), num_tokens, prompt_len=64, device=dev,
                                         repeats=5):
        out[f"batch {r['batch_size']}"] = {
            "new_tokens": r["num_tokens"], "prompt_len": r["prompt_len"], "timed_runs": r["df11"]["timed_runs"],
            "bf16_tokens_per_second": r["bf16"]["tokens_per_second"],
            "df11_tokens_per_second": r["df11"]["tokens_per_second"],
            "df11_over_bf16": r["df11_over_bf16_tokens_per_second"],
            "bf16_peak_memory_mb": r["bf16"]["gpu_peak_memory_mb"],
            "df11_peak_memory_mb": r["df11"]["gpu_peak_memory_mb"],
            "logits_bit_identical": r["logits_bit_identical"], "tokens_identical": r["tokens_identical"]}
        out["model"] = r["model"]
        out["compressed_over_bf16"] = r["compressed_over_bf16"]
        out["compress_seconds_host"] = r["compress_seconds"]
    out["leg_seconds"] = time.perf_counter() - t0
    return out


def offload(torch, dev, double_blocks, single_blocks):
    """One pass over a FLUX.1-dev-shaped block stack (hidden 3072, 4096 image + 512 text
    tokens) in BF16, with resident DF11 streams, and with the streams in pinned host memory
    copied one block ahead of use (cpu_offload): time per pass, peak device memory, what a
    block costs when nothing overlaps (host-to-device copy, then decode), how well the copies
    overlap, and whether the outputs are identical."""
    import types

    import bench_extra
    t0 = time.perf_counter()
    a = types.SimpleNamespace(double_blocks=double_blocks, single_blocks=single_blocks, image_tokens=4096,
                              text_tokens=512)
    r = bench_extra.flux_report(a, torch, dev, passes=6)
    out = {"double_blocks": double_blocks, "single_blocks": single_blocks, "hidden": 3072,
           "image_tokens": 4096, "text_tokens": 512, "parameters": r["config"]["parameters"]}
    for key, run in r["passes"].items():
        out[key] = {"ms_per_pass": run["steady_pass_s"] * 1e3, "peak_device_memory_mb": run["peak_device_memory_mb"]}
    out["per_block_unoverlapped"] = [
        {"block": b["block"], "n_elements": b["n_elements"], "host_to_device_ms": b["h2d_ms"],
         "host_to_device_GBps": b["h2d_GBps"], "decode_ms": b["decode_ms"]} for b in r["per_block_serial"]]
    out["overlap_efficiency"] = r["overlap_efficiency"]
    out["outputs_bit_identical"] = r["outputs_bit_identical"]
    out["leg_seconds"] = time.perf_counter() - t0
    return out


def profiled_traffic():
    """HBM bytes per launch of decode_kernel on this workload, as the committed
    counter summary recorded them (FETCH_SIZE and WRITE_SIZE passes, each scaled
    by what the same counter reads for a plain copy of known size).  Counters
    cannot be read from inside this process, so None when the summary is absent."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                        "decode_kernel_llama3_8b_block.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch"):
                return int(line.split("=")[1])
    except OSError:
        pass
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--preheat-ms", type=float, default=400.0,
                    help="decode launches for this long before the counted warm-up, so that the timed steps "
                         "run at the clock the device settles at under load, whatever --warmup is")
    ap.add_argument("--no-mixes", action="store_true",
                    help="skip the per-distribution and per-size side measurements (config.mixes, config.sizes)")
    ap.add_argument("--no-embedding-mixes", action="store_true",
                    help="config.mixes on the 4096x14336 matrix only, not on the 151936x4096 tensor as well, and no config.rows")
    ap.add_argument("--no-e2e", action="store_true",
                    help="skip config.e2e: Qwen3-8B-shaped generation, BF16 against DF11, batch 1 and 64 (about 1 min)")
    ap.add_argument("--e2e-tokens", type=int, default=64, help="new tokens per sequence in config.e2e")
    ap.add_argument("--no-offload", action="store_true",
                    help="skip config.offload: FLUX-shaped block stack with cpu_offload (about 20 s)")
    ap.add_argument("--offload-blocks", type=int, nargs=2, default=(4, 8), metavar=("DOUBLE", "SINGLE"),
                    help="double-stream and single-stream blocks of the config.offload stack (the full model: 19 38)")
    ap.add_argument("--copies", type=int, default=4,
                    help="device copies of the compressed block that the steps decode in turn")
    ap.add_argument("--timed-only", action="store_true",
                    help="after the timed region, skip the two extra passes over the same workload (an event pair "
                         "around every launch; one and the same copy over and over): under a profiler every "
                         "decode launch of the run is then of one kind")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run a 256 MiB streaming copy kernel 5 times (profiler byte-counter calibration)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU only: every box has one MI355X and the decode path "
                 "needs no exchange between GPUs; run with --gpus 1")

    import torch
    from dfloat11_amd import decode as D
    from dfloat11_amd import dfloat11_utils as U

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    w = make_block(torch, dev)
    n_elements = w.numel()
    w_cpu = w.cpu()
    t0 = time.perf_counter()
    codec, _ = U.get_codec(w_cpu)
    luts = U.get_luts(codec.get_code_table())
    enc, sm, pos, gaps, _ = U.encode_weights([w_cpu], codec)
    t_encode = time.perf_counter() - t0
    pos_np = pos.numpy().astype(np.int64)
    max_elems = int((pos_np[1:] - pos_np[:-1]).max())

    # The compressed block is held in `a.copies` separate device copies and successive
    # steps decode them in turn, into one output buffer, the way the blocks of a model
    # follow each other: 4 x 295 MB of compressed input is more than the 256 MB of
    # memory-side cache, so every step reads its input from HBM.  (Decoding one and the
    # same copy over and over is several per cent faster: `same_input_kernel_ms_median`
    # in the result.)
    from dfloat11_amd import _native
    lib = _native.hip_lib()
    out = torch.empty(n_elements, dtype=torch.bfloat16, device=dev)
    stream_handle = torch.cuda.current_stream(dev).cuda_stream
    copies = []
    prepare_ms = []
    for _ in range(max(1, a.copies)):
        d_luts, d_enc, d_sm, d_gaps = (t.to(dev) for t in (luts, enc, sm, gaps))
        d_pos = pos.view(torch.uint8).to(dev)
        # load-time step, once per compressed module: layout check on the host, then decode
        # tables and sub-block positions on the device (not part of a decode)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        D.validate_stream(d_luts, d_enc, d_sm, d_pos, d_gaps)
        t1 = time.perf_counter()
        ws, max_sub = D.prepare(d_luts, d_enc, d_pos, d_gaps, n_elements)   # waits for its kernels
        t2 = time.perf_counter()
        prepare_ms.append(((t1 - t0) * 1e3, (t2 - t1) * 1e3))
        D.decode(d_luts, d_enc, d_sm, d_pos, d_gaps, out, ws, max_sub)   # once through the checked wrapper
        # One step = one call of the C-ABI entry point on torch's current stream, with the
        # arguments bound once (the Python wrapper's checks stay out of the timed region).
        copies.append(((d_luts, d_enc, d_sm, d_gaps, d_pos, ws),
                       (d_luts.data_ptr(), d_enc.data_ptr(), d_sm.data_ptr(), d_pos.data_ptr(), d_gaps.data_ptr(),
                        out.data_ptr(), int(luts.shape[0]), int(enc.numel()), int(n_elements), ws.data_ptr(),
                        int(max_sub), stream_handle)))
    counter = [0]

    def step():
        rc = lib.df11_decode(*copies[counter[0] % len(copies)][1])
        counter[0] += 1
        if rc != 0:
            raise RuntimeError(f"df11_decode failed: {rc}")

    # Pre-heat by time: the first launches after idle run at a lower clock (about 60 launches
    # on this device); the counted warm-up follows.
    t0 = time.perf_counter()
    preheat_launches = 0
    while (time.perf_counter() - t0) * 1e3 < a.preheat_ms:
        for _ in range(16):
            step()
        preheat_launches += 16
        torch.cuda.synchronize()
    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    if a.calibration_copy:
        import ctypes
        from dfloat11_amd import build as B
        copy_lib = ctypes.CDLL(B.CALIBRATION_LIB)   # built by build(); not part of the decode library
        copy_lib.calibration_copy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        src = torch.zeros(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            rc = copy_lib.calibration_copy(src.data_ptr(), dst.data_ptr(), src.numel(), stream_handle)
            if rc != 0:
                raise RuntimeError(f"calibration_copy failed: {rc}")
        torch.cuda.synchronize()
        del src, dst
    # The timed region: K steps launched back to back, between two HIP events on the
    # stream the kernel is launched on (torch's current stream) and a device
    # synchronisation on either side.  A step is one launch, so the region's length
    # over K is the average launch duration with the gaps between launches counted in.
    region_start, region_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    region_start.record()
    for i in range(a.steps):
        step()
    region_end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    span_ms = region_start.elapsed_time(region_end)
    ms_per_step = span_ms / a.steps
    avg_kernel_ms = ms_per_step
    # The same K steps again with an event pair around every launch, for the spread.  The
    # events between launches lengthen both the step (by about 7 us) and the interval they
    # measure (by about 2 us), so these figures are reported beside the region's, not used.
    kernel_ms, same_ms = [ms_per_step], None
    if not a.timed_only:
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(a.steps)]
        ends = [torch.cuda.Event(enable_timing=True) for _ in range(a.steps)]
        for i in range(a.steps):
            starts[i].record()
            step()
            ends[i].record()
        torch.cuda.synchronize()
        kernel_ms = [s.elapsed_time(e) for s, e in zip(starts, ends)]

        # the same measurement with every step decoding the same copy (inputs may stay in cache)
        same = []
        for i in range(60 + 40):
            s0, e0 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s0.record()
            lib.df11_decode(*copies[0][1])
            e0.record()
            if i >= 60:
                same.append((s0, e0))
        torch.cuda.synchronize()
        same_ms = float(np.median([s0.elapsed_time(e0) for s0, e0 in same]))

    bit_exact = None
    if not a.no_verify:
        bit_exact = bool(torch.equal(out.view(torch.int16), w.view(torch.int16)))

    n_bytes = enc.numel()
    algo = algorithmic_bytes(n_bytes, n_elements, luts.shape[0])
    value = algo / (ms_per_step * 1e-3) / 1e9
    achieved = algo / (avg_kernel_ms * 1e-3) / 1e9

    result = {
        "metric": "decode GB/s (bytes in+out)", "value": value, "unit": "GB/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8",
        "data": "synthetic",
        "config": {
            "workload": "Llama-3-8B-shaped decoder block (q,k,v,o,gate,up,down) as one DF11 stream, "
                        "random-init N(0,0.02) BF16, decoded into one contiguous buffer; successive steps read "
                        "different device copies of the compressed block",
            "n_elements": n_elements, "encoded_exponent_bytes": n_bytes,
            "bitstream_blocks": -(-n_bytes // 4096), "n_luts": int(luts.shape[0]),
            "algorithmic_bytes_per_step": algo, "bytes_per_element": algo / n_elements,
            "compressed_over_bf16": (n_bytes + n_elements + gaps.numel() + 4 * pos.numel()) / (2 * n_elements),
            "max_elems_per_block": max_elems, "max_elems_per_subblock": max_sub,
            "workspace_bytes": int(ws.numel()), "bit_exact": bit_exact,
            "encode_seconds_host": t_encode, "wall_ms_per_step": wall * 1e3 / a.steps,
            "kernel_ms_min": float(np.min(kernel_ms)), "kernel_ms_max": float(np.max(kernel_ms)),
            "kernel_ms_median": float(np.median(kernel_ms)), "kernel_ms_mean": float(np.mean(kernel_ms)),
            "input_copies_decoded_in_turn": len(copies), "same_input_kernel_ms_median": same_ms,
            "preheat_ms": a.preheat_ms, "preheat_launches": preheat_launches,
            # first-use cost of a compressed module (median over the copies; the first call also
            # loads the library's code object): host-side layout check + df11_prepare incl. its wait
            "prepare_ms": float(np.median([v + p for v, p in prepare_ms])),
            "prepare_ms_validate_stream": float(np.median([v for v, _ in prepare_ms])),
            "prepare_ms_df11_prepare": float(np.median([p for _, p in prepare_ms])),
        },
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": profiled_traffic(),
                     "kernel": "decode_kernel_" + lib.df11_launch_plan_name(
                         int(n_bytes), int(n_elements),
                         torch.cuda.get_device_properties(dev).multi_processor_count).decode().replace("/", "_"),
                     "avg_launch_ms": avg_kernel_ms},
    }
    if not a.no_mixes:
        copies.clear()
        out = None
        torch.cuda.empty_cache()
        result["config"]["mixes"], result["config"]["sizes"] = side_measurements(
            torch, dev, embedding_shape=not a.no_embedding_mixes)
        if not all(m["bit_exact"] for m in list(result["config"]["mixes"].values())
                   + list(result["config"]["sizes"].values())):
            result["error"] = "a side measurement did not decode bit-exactly"
            bit_exact = False
        if not a.no_embedding_mixes:
            # the embedding's lookup: only the rows of the ids (df11_decode_rows) against the whole table
            import bench_extra
            result["config"]["rows"] = rows = bench_extra.measure_rows(torch, dev, row_counts=(1, 64, 4096))
            torch.cuda.empty_cache()
            if not all(r["bit_exact"] for r in rows):
                result["error"] = "a row decode differs from the original rows"
                bit_exact = False
    if not a.no_cpu_baseline:
        stream = dict(luts=luts.numpy(), encoded_exponent=enc.numpy(), sign_mantissa=sm.numpy(),
                      output_positions=pos.numpy(), gaps=gaps.numpy())
        result["cpu_baseline"] = cpu_baseline(stream, w_cpu.view(torch.int16).numpy().view(np.uint16))
        if not result["cpu_baseline"]["bit_exact"]:
            result["error"] = "the CPU oracle's output differs from the original block"
            bit_exact = False
    copies.clear()
    out = None
    torch.cuda.empty_cache()
    if not a.no_e2e:
        result["config"]["e2e"] = e2e = end_to_end(torch, dev, a.e2e_tokens)
        if not all(v["logits_bit_identical"] and v["tokens_identical"] for k, v in e2e.items() if k.startswith("batch")):
            result["error"] = "DF11 generation differs from BF16"
            bit_exact = False
    if not a.no_offload:
        result["config"]["offload"] = off = offload(torch, dev, *a.offload_blocks)
        if not all(off["outputs_bit_identical"].values()):
            result["error"] = "offloaded pass differs from the resident one"
            bit_exact = False
    if bit_exact is False and "error" not in result:
        result["error"] = "decoded block differs from the original"
    print(json.dumps(result))
    if bit_exact is False:
        sys.exit(1)


if __name__ == "__main__":
    main()
