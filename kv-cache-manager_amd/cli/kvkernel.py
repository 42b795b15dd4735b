"""kvkernel: the decode attention kernels alone, over a grid of context lengths, batch sizes and
page sizes, with the reference tool's flags and columns (src/main_kernel_bench.cpp:34-126):

  --ctx 128,256,512,1024,2048  --batch 1,8,32,128  --block-size 16  --heads 32  --kv-heads 4
  --head-dim 64  --iters 100  --out FILE.csv  [--graph]

Six variants per point: v1 (one pass over the context per row and head), v2 (contexts cut into
partitions that run in parallel and are merged) and, not in the reference, "fused" (the kernel
decode steps run: one launch that also takes q, k, v from the projection and writes the new key
and value to their page), each through a shuffled block table ("paged") and through a table of
consecutive pages ("contiguous").  5 warm-up calls, then
``--iters`` timed calls between two events; GB/s = 2 * batch * ctx * kv_heads * head_dim * 2 bytes
/ time, the keys and values a call has to read once.  Zero-filled bfloat16 cache, scale 0.125.
With --graph (not in the reference) the timed calls are replays of one captured HIP graph that
holds ``--iters`` calls, which takes the host's launch cost out of the figure.
Columns: registers per lane, LDS per workgroup, workgroups per CU, occupancy (resident waves as a
percentage of a CU's 32 wave slots), workgroups launched and how many rounds of the chip they make.

  --prefill 2048,1024,512@1536  [--seqs 1]        (not in the reference)

times the tiled prompt attention instead: each item is a portion of TOKENS query rows that starts
at position START of its sequence (default 0), ``--seqs`` such sequences in one call; random keys
and values behind a shuffled block table.  TFLOP/s counts the causal work, 4 * head_dim * heads *
(keys each row sees), against the bf16 matrix-core peak; the last columns say how the launch was
cut (query rows per workgroup, keys per segment).

  --floor [--nodes 156]                          (not in the reference)

times what a launch costs and how fast memory streams inside a chain of dependent launches like a
decode step's: ``--nodes`` launches of one probe kernel after the other, as plain stream launches and
as one captured HIP graph: an empty kernel (1 and 1,024 workgroups), a kernel that reads what the one
before it wrote (64 KB, 1 MB), and kernels that stream 8, 23 and 46 MB each from a 2 GiB buffer (the
sizes of a TinyLlama layer's weight matrices; consecutive launches read consecutive regions, so that
the bytes come from HBM and not from a cache).

  --sync [--layers 22]                           (not in the reference)

times what it costs the workgroups of ONE launch to depend on one another, the alternative to a chain of
launches: a barrier across the launch (data handed over by stores and loads past the caches, or by fences),
split sums added up by the last workgroup of a tile to arrive against a second launch that adds them, and the
bytes of a whole decode step (``--layers`` layers of five phases at TinyLlama sizes) read by one launch whose
phases wait for one another against one launch per phase.  Every wait inside these kernels is bounded.
"""
import sys

import numpy as np

from .args import Args

PEAK_GBS = 8000.0      # MI355X HBM3E
PEAK_BF16_TFLOPS = 2500.0
WAVE_SLOTS_PER_CU = 32


def _floor(nodes):
    import torch
    from .. import ops
    ops.lib()
    dev = torch.device("cuda:0")
    big = torch.zeros(1 << 29, dtype=torch.int32, device=dev)            # 2 GiB
    ping, pong = torch.zeros(1 << 18, dtype=torch.int32, device=dev), torch.zeros(1 << 18, dtype=torch.int32, device=dev)
    sink = torch.zeros(256, dtype=torch.float32, device=dev)
    total = big.numel() * 4

    def chain_empty(grid, block):
        return lambda i: ops.probe_empty(grid, block)

    def chain_touch(nbytes, grid):
        n = nbytes // 4
        return lambda i: ops.probe_copy(ping[:n] if i % 2 == 0 else pong[:n], pong[:n] if i % 2 == 0 else ping[:n], grid=grid)

    def chain_stream(nbytes, grid):
        n = nbytes // 4
        def launch(i):
            lo = (i * n) % (big.numel() - n)
            lo -= lo % 4
            ops.probe_read(big[lo:lo + n], sink, grid=grid)
        return launch

    cases = [("empty <<<1,64>>>", chain_empty(1, 64), 0), ("empty <<<1024,256>>>", chain_empty(1024, 256), 0),
             ("reads what the last wrote, 64 KB", chain_touch(64 << 10, 16), 0),
             ("reads what the last wrote, 1 MB", chain_touch(1 << 20, 256), 0),
             ("streams 8 MB", chain_stream(8 << 20, 512), 8 << 20), ("streams 23 MB", chain_stream(23 << 20, 1024), 23 << 20),
             ("streams 46 MB", chain_stream(46 << 20, 1024), 46 << 20)]
    print(f"{nodes} launches in a row; microseconds per launch")
    print("%-36s %10s %10s %12s" % ("kernel", "stream", "graph", "graph TB/s"))
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for name, launch, nbytes in cases:
            def run_all():
                for i in range(nodes):
                    launch(i)
            run_all()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            stream.synchronize()
            e0.record()
            for _ in range(10):
                run_all()
            e1.record()
            e1.synchronize()
            eager = 1e3 * e0.elapsed_time(e1) / (10 * nodes)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                run_all()
            for _ in range(3):
                graph.replay()
            stream.synchronize()
            e0.record()
            for _ in range(30):
                graph.replay()
            e1.record()
            e1.synchronize()
            g = 1e3 * e0.elapsed_time(e1) / (30 * nodes)
            rate = "%.2f" % (nbytes / g / 1e6) if nbytes else ""
            print("%-36s %10.2f %10.2f %12s" % (name, eager, g, rate))
        # what a launch streams as a function of the CUs it covers and the waves on each: 46 MB (a gate/up matrix of
        # TinyLlama sizes), every workgroup a contiguous share, consecutive launches consecutive regions
        n = (46 << 20) // 4
        print("\n46 MB read by one launch of G workgroups of W waves (a contiguous share each, 8 loads of 16 bytes on their"
              "\nway per lane; 16 where said), launches of a graph one after the other: microseconds, TB/s")
        print("%6s %4s %10s %10s" % ("G", "W", "us", "TB/s"))
        for G, W, inflight in ((64, 4, 8), (128, 4, 8), (176, 4, 8), (176, 8, 8), (176, 4, 16), (235, 3, 8), (256, 2, 8), (256, 4, 8),
                               (256, 8, 8), (512, 4, 8), (1024, 4, 8)):
            def run_all():
                for i in range(16):
                    lo = (i * n) % (big.numel() - n)
                    lo -= lo % 4
                    ops.probe_stream(big[lo:lo + n], sink, G, W, inflight)
            run_all()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                run_all()
            for _ in range(3):
                graph.replay()
            stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(20):
                graph.replay()
            e1.record()
            e1.synchronize()
            us = 1e3 * e0.elapsed_time(e1) / (20 * 16)
            print("%6d %4d %10.2f %10.2f%s" % (G, W, us, n * 4 / us / 1e6, "   (16 loads per lane)" if inflight == 16 else ""))
    return 0


def _sync(layers):
    """What it costs workgroups of one launch to depend on one another, against what launches cost:
    a barrier across the launch, split sums added by the last workgroup to arrive or by a second launch,
    and a decode step's bytes read by one launch of dependent phases or by one launch per phase."""
    import torch
    from .. import ops
    ops.lib()
    dev = torch.device("cuda:0")
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    flags = torch.zeros(2, dtype=torch.int32, device=dev)
    stream = torch.cuda.Stream()

    def timed(fn, reps=20, calls=1):
        """Microseconds per call of fn; ``calls`` calls in a row make one captured graph, which is replayed."""
        with torch.cuda.stream(stream):
            fn()
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for _ in range(calls):
                    fn()
            for _ in range(2):
                graph.replay()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            stream.synchronize()
            e0.record()
            for _ in range(reps):
                graph.replay()
            e1.record()
            e1.synchronize()
        return 1e3 * e0.elapsed_time(e1) / (reps * calls)

    print(f"{cus} CUs.  A barrier across the workgroups of one launch (microseconds per barrier, from 1 and 101 rounds):")
    data = torch.zeros(2 * 1024 * 256, dtype=torch.float32, device=dev)
    counter = torch.zeros(1, dtype=torch.int32, device=dev)
    print("%-44s %12s %12s" % ("data handed over by", "64 workgroups", f"{cus} workgroups"))
    for fences, label in ((False, "stores and loads past the caches"), (True, "release and acquire fences")):
        row = []
        for G in (64, cus):
            def go(rounds):
                return timed(lambda: (counter.zero_(), ops.probe_barrier(data, counter, flags, G, rounds, fences=fences)))
            row.append((go(101) - go(1)) / 100.0)
        print("%-44s %12.2f %12.2f" % (label, *row))
    print()
    print("Split sums (4 KB per workgroup) added up by the tile's last workgroup to arrive, or by a second launch (microseconds):")
    print("%8s %8s %16s %16s %16s" % ("splits", "tiles", "last arriver", "two launches", "an empty launch"))
    partials = torch.zeros(8 * 512 * 1024, dtype=torch.float32, device=dev)
    out = torch.zeros(512 * 1024, dtype=torch.float32, device=dev)
    counters = torch.zeros(512, dtype=torch.int32, device=dev)
    for S in (4, 8):
        for tiles in (32, 128, 512):
            a = timed(lambda: ops.probe_sums(partials, counters, out, S, tiles, True, flags), 20, calls=40)
            b = timed(lambda: ops.probe_sums(partials, counters, out, S, tiles, False, flags), 20, calls=40)
            c = timed(lambda: ops.probe_empty(tiles * S, 256), 20, calls=40)
            print("%8d %8d %16.2f %16.2f %16.2f" % (S, tiles, a, b, c))
    print()
    # a layer of TinyLlama-1.1B sizes: QKV, the cache of eight requests, O, gate and up, down
    H, I, QKV = 2048, 5632, 2560
    phases = [QKV * H * 2, 1 << 20, H * H * 2, 2 * I * H * 2, H * I * 2]
    layer = sum(phases)
    weights = torch.zeros(4 * layer // 4, dtype=torch.int32, device=dev)
    act = torch.zeros(8192, dtype=torch.float32, device=dev)
    sink = torch.zeros(1024, dtype=torch.int32, device=dev)
    cnt = torch.zeros(layers * len(phases) * 17, dtype=torch.int32, device=dev)
    total = layer * layers
    print(f"A decode step's bytes ({layers} layers of {len(phases)} phases, {total / 1e9:.2f} GB) read by:")
    one = timed(lambda: (cnt.zero_(), ops.probe_phases(weights, phases, layers, True, cus, cnt, act, flags, sink)), 10)
    chain = timed(lambda: ops.probe_phases(weights, phases, layers, False, sink=sink), 10)
    whole = timed(lambda: ops.probe_read(weights, sink, grid=2048), 10) * total / (4 * layer)
    print("%-64s %10.1f us %8.2f TB/s" % (f"one launch of {cus} workgroups, a phase waits for the one before", one, total / one / 1e6))
    print("%-64s %10.1f us %8.2f TB/s" % (f"one launch per phase ({layers * len(phases)} graph nodes)", chain, total / chain / 1e6))
    print("%-64s %10.1f us %8.2f TB/s" % ("one launch that depends on nothing (scaled from four layers)", whole, total / whole / 1e6))
    gave_up, wrong = [int(v) for v in flags.cpu()]
    print(f"workgroups that gave up waiting: {gave_up}; wrong values read: {wrong}")
    return 1 if (gave_up or wrong) else 0


def _ints(s):
    return [int(x) for x in s.split(",") if x]


def main(argv=None):
    a = Args(sys.argv[1:] if argv is None else argv)
    ctxs, batches, blocks = _ints(a.str("ctx", "128,256,512,1024,2048")), _ints(a.str("batch", "1,8,32,128")), _ints(a.str("block-size", "16"))
    heads, kvh, hd = a.i32("heads", 32), a.i32("kv-heads", 4), a.i32("head-dim", 64)
    iters, out_csv = a.i32("iters", 100), a.str("out", "")
    use_graph = a.flag("graph")
    prefill, seqs = a.str("prefill", ""), a.i32("seqs", 1)
    floor, nodes = a.flag("floor"), a.i32("nodes", 156)
    sync, layers = a.flag("sync"), a.i32("layers", 22)
    a.warn_unused()
    if prefill:
        return _prefill(prefill, seqs, blocks, heads, kvh, hd, iters, out_csv, use_graph)
    if floor:
        return _floor(nodes)
    if sync:
        return _sync(layers)

    import torch
    from .. import ops
    ops.lib()
    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(dev)
    cus = props.multi_processor_count
    print(f"device {props.name}, {cus} CUs, peak HBM bandwidth {PEAK_GBS:.1f} GB/s")
    f = open(out_csv, "w") if out_csv else None
    if f:
        f.write("block_size,batch,ctx,variant,us,gbps,pct_peak,regs,lds_bytes,wgs_per_cu,occupancy_pct,wgs,rounds\n")
    print("%5s %6s %6s %-16s %10s %9s %7s %5s %7s %6s %6s %7s" % ("B", "batch", "ctx", "variant", "us/call", "GB/s",
                                                                   "%peak", "regs", "lds", "wg/CU", "occ%", "rounds"))
    rng = np.random.default_rng(0)
    bf16 = torch.bfloat16
    for B in blocks:
        for batch in batches:
            for ctx in ctxs:
                mb = (ctx + B - 1) // B
                nb = batch * mb
                K = torch.zeros(nb, kvh, B, hd, dtype=bf16, device=dev)
                V = torch.zeros(nb, kvh, hd, B, dtype=bf16, device=dev)
                Q = torch.zeros(batch, heads * hd, dtype=bf16, device=dev)
                O = torch.zeros(batch, heads * hd, dtype=bf16, device=dev)
                seq_tab = np.arange(nb, dtype=np.int32)
                tables = {"paged": torch.tensor(rng.permutation(seq_tab), device=dev),
                          "contiguous": torch.tensor(seq_tab, device=dev)}
                rows = torch.arange(batch, dtype=torch.int32, device=dev)
                lens = torch.full((batch,), ctx, dtype=torch.int32, device=dev)
                v2_ok = ops.attention_decode_supported(heads, kvh, hd, bf16, B)
                scratch = (torch.zeros(ops.attention_decode_scratch(batch, heads, hd, ctx), dtype=torch.float32, device=dev)
                           if v2_ok else None)
                nbytes = 2.0 * batch * ctx * kvh * hd * 2

                def v1(tab):
                    ops.attention(Q, O, K, V, tab, mb, rows, lens, heads, kvh, hd, 0.125)

                def v2(tab):
                    ops.attention_decode(Q, O, K, V, tab, mb, rows, lens, heads, kvh, hd, 0.125, ctx, scratch)

                fused_ok = ops.attention_decode_fused_supported(heads, kvh, hd, bf16, B)
                QKV = torch.zeros(batch, (heads + 2 * kvh) * hd, dtype=bf16, device=dev)
                slots = {k: (t.view(batch, mb)[:, (ctx - 1) // B] * B + (ctx - 1) % B).to(torch.int32).contiguous()
                         for k, t in tables.items()}

                fneed = ops.attention_decode_fused_scratch(batch, heads, kvh, hd, ctx) if fused_ok else 0
                fscratch = torch.zeros(fneed, dtype=torch.float32, device=dev) if fneed else None

                def fused(tab):
                    ops.attention_decode_fused(QKV, O, K, V, tab, mb, rows, lens, heads, kvh, hd, 0.125,
                                               slots=slots["paged" if tab is tables["paged"] else "contiguous"],
                                               max_context=ctx, scratch=fscratch)

                for version, call in (("v1", v1), ("v2", v2), ("fused", fused)):
                    for layout in ("paged", "contiguous"):
                        name = f"{layout}-{version}"
                        if (version == "v2" and not v2_ok) or (version == "fused" and not fused_ok):
                            print("%5d %6d %6d %-16s %10s" % (B, batch, ctx, name, "unsupported"))
                            continue
                        tab = tables[layout]
                        for _ in range(5):
                            call(tab)
                        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        if use_graph:
                            torch.cuda.synchronize()
                            graph = torch.cuda.CUDAGraph()
                            with torch.cuda.graph(graph):
                                for _ in range(iters):
                                    call(tab)
                            graph.replay()
                            torch.cuda.synchronize()
                            e0.record()
                            graph.replay()
                            e1.record()
                        else:
                            e0.record()
                            for _ in range(iters):
                                call(tab)
                            e1.record()
                        e1.synchronize()
                        us = 1e3 * e0.elapsed_time(e1) / iters
                        gbs = nbytes / (us * 1e-6) / 1e9
                        info = ops.attention_kernel_info(version, heads, kvh, hd)
                        waves = info["threads"] // 64
                        occ = 100.0 * info["workgroups_per_cu"] * waves / WAVE_SLOTS_PER_CU
                        wgs = ((batch * heads + 3) // 4 if version == "v1"
                               else kvh * batch * ((ctx + 255) // 256) if version == "v2" else kvh * batch)
                        rounds = wgs / float(max(info["workgroups_per_cu"], 1) * cus)
                        print("%5d %6d %6d %-16s %10.2f %9.1f %6.1f%% %5d %6dB %6d %5.0f%% %7.2f" % (
                            B, batch, ctx, name, us, gbs, 100 * gbs / PEAK_GBS, info["regs"], info["lds_bytes"],
                            info["workgroups_per_cu"], occ, rounds))
                        if f:
                            f.write("%d,%d,%d,%s,%.3f,%.2f,%.2f,%d,%d,%d,%.1f,%d,%.3f\n" % (
                                B, batch, ctx, name, us, gbs, 100 * gbs / PEAK_GBS, info["regs"], info["lds_bytes"],
                                info["workgroups_per_cu"], occ, wgs, rounds))
    if f:
        f.close()
    return 0


def _prefill(spec, seqs, blocks, heads, kvh, hd, iters, out_csv, use_graph):
    import torch
    from .. import ops
    ops.lib()
    dev = torch.device("cuda:0")
    bf16 = torch.bfloat16
    items = []
    for part in spec.split(","):
        tokens, _, start = part.partition("@")
        items.append((int(tokens), int(start or 0)))
    f = open(out_csv, "w") if out_csv else None
    if f:
        f.write("block_size,seqs,tokens,start,us,tflops,pct_peak,tile_rows,segment\n")
    print("%5s %5s %7s %7s %10s %9s %7s %5s %8s" % ("B", "seqs", "tokens", "start", "us/call", "TFLOP/s", "%peak", "rows", "segment"))
    gen = torch.Generator(device=dev).manual_seed(0)
    for B in blocks:
        if not ops.attention_prefill_supported(heads, kvh, hd, bf16, B):
            print("%5d %s" % (B, "unsupported"))
            continue
        for tokens, start in items:
            ctx = start + tokens
            mb = (ctx + B - 1) // B
            K = torch.randn(seqs * mb, kvh, B, hd, device=dev, generator=gen).to(bf16)
            V = torch.randn(seqs * mb, kvh, hd, B, device=dev, generator=gen).to(bf16)
            Q = torch.randn(seqs * tokens, (heads + 2 * kvh) * hd, device=dev, generator=gen).to(bf16)
            O = torch.zeros(seqs * tokens, heads * hd, dtype=bf16, device=dev)
            tab = torch.randperm(seqs * mb, device=dev, generator=gen).to(torch.int32)
            run_start = torch.arange(0, seqs * tokens + 1, tokens, dtype=torch.int32, device=dev)
            seq_start = torch.full((seqs,), start, dtype=torch.int32, device=dev)
            need = ops.attention_prefill_scratch(seqs * tokens, heads, hd, ctx, tokens, seqs)
            scratch = torch.zeros(max(need, 4), dtype=torch.float32, device=dev)

            def call():
                ops.attention_prefill(Q, O, K, V, tab, mb, run_start, seq_start, seqs, tokens, heads, kvh, hd,
                                      1.0 / hd ** 0.5, rows=seqs * tokens, max_context=ctx, scratch=scratch)

            for _ in range(5):
                call()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            if use_graph:
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    for _ in range(iters):
                        call()
                graph.replay()
                torch.cuda.synchronize()
                e0.record()
                graph.replay()
                e1.record()
            else:
                e0.record()
                for _ in range(iters):
                    call()
                e1.record()
            e1.synchronize()
            us = 1e3 * e0.elapsed_time(e1) / iters
            seen = seqs * (tokens * start + tokens * (tokens + 1) / 2.0)
            tflops = 4.0 * hd * heads * seen / (us * 1e-6) / 1e12
            rows = ops.attention_prefill_tile_rows(seqs * tokens, heads, hd, ctx, tokens, seqs)
            seg = ops.attention_prefill_segment(seqs * tokens, heads, hd, ctx, tokens, seqs)
            print("%5d %5d %7d %7d %10.2f %9.1f %6.1f%% %5d %8d" % (B, seqs, tokens, start, us, tflops,
                                                                  100 * tflops / PEAK_BF16_TFLOPS, rows, seg))
            if f:
                f.write("%d,%d,%d,%d,%.3f,%.2f,%.2f,%d,%d\n" % (B, seqs, tokens, start, us, tflops,
                                                               100 * tflops / PEAK_BF16_TFLOPS, rows, seg))
    if f:
        f.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
