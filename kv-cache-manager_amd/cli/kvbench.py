"""kvbench: serve a synthetic workload and report throughput and latency.

  kvbench --model DIR | --random-weights [--sizes tinyllama-1.1b] \\
          [--policy paged|contiguous] [--pool-gb 1] [--requests 500] [--rate 8] [--summary out.csv]

Requests arrive by a Poisson process in wall-clock time (--rate req/s, 0 = all at once).  Token
ids are random.  Flags and defaults follow the reference's kvbench (src/main_bench.cpp:21-131)."""
import math
import sys
import time

from .args import Args
from .common import engine_config_from_args, make_engine


def main(argv=None):
    try:
        a = Args(sys.argv[1:] if argv is None else argv)
        ec = engine_config_from_args(a)
        from ..engine.metrics import BenchSummary, MetricsCollector, append_bench_csv, print_summary
        from ..engine.workload import WorkloadConfig, generate_workload, make_prompt_tokens
        wl = WorkloadConfig.from_args(a)
        wl.max_seq_len = ec.max_seq_len
        warmup = a.i32("warmup", 8)
        summary_csv, step_log = a.str("summary", ""), a.str("step-log", "")
        time_limit = a.f64("time-limit", 1e9)
        temperature, sampler_seed = a.f64("temperature", 0.0), a.i64("sampler-seed", 0)
        eng = make_engine(a, ec)
        wl.max_seq_len = eng.config.max_seq_len      # as built: within the model's own range
        a.warn_unused()
        wl.vocab = eng.model.spec.vocab_size
        import torch
        print(f"weights {eng.runner.weight_bytes / 2**30:.2f} GB, KV pool {eng.num_blocks} blocks x {eng.bytes_per_block()} B = "
              f"{eng.cache_bytes() / 2**30:.2f} GB")

        # warm-up: a few short requests run to completion (kernel loading, graph capture)
        w = WorkloadConfig(**{**wl.__dict__, "num_requests": warmup, "arrival_rate": 0.0, "shared_frac": 0.0,
                              "seed": wl.seed + 999, "min_output": 16, "max_output": 16, "output_sigma": 0.0,
                              "output_mu": math.log(16.0)})
        for r in generate_workload(w):
            eng.add_request(make_prompt_tokens(r, w), r.output_len, request_id=10_000_000 + r.id)
        eng.run_until_idle()
        eng.core.reset_counters()
        ps0 = eng.core.prefix_stats()

        reqs = generate_workload(wl)
        print(wl.describe())
        log = open(step_log, "w") if step_log else None
        if log:
            log.write("t,rows,seqs,prefill_tokens,decode_seqs,ms,running,waiting,blocks_in_use\n")
        mc, s = MetricsCollector(), BenchSummary()
        nxt, step_ms_sum, rejected = 0, 0.0, 0
        eng.reset_clock()
        while mc.count() + rejected < len(reqs):
            now = eng.now()
            if now > time_limit:
                print("time limit reached")
                break
            while nxt < len(reqs) and reqs[nxt].arrival <= now:
                r = reqs[nxt]
                eng.add_request(make_prompt_tokens(r, wl), r.output_len, temperature, sampler_seed, request_id=r.id,
                                arrival=r.arrival)
                nxt += 1
            if eng.idle():
                if nxt < len(reqs):
                    time.sleep(max(0.0, reqs[nxt].arrival - eng.now()))
                continue
            si = eng.step()
            step_ms_sum += si.ms
            s.peak_blocks = max(s.peak_blocks, eng.core.blocks_in_use())
            if log:
                log.write(f"{eng.now():.4f},{si.rows},{si.seqs},{si.prefill_tokens},{si.decode_seqs},{si.ms:.3f},"
                          f"{eng.core.num_running()},{eng.core.num_waiting()},{eng.core.blocks_in_use()}\n")
            for f in eng.take_finished():
                rejected += f.rejected
                mc.add_finished(f)
        wall = eng.now()
        if log:
            log.close()
        c = eng.core.counters()
        s.policy, s.block_size, s.num_blocks = eng.core.name, ec.block_size, eng.num_blocks
        s.pool_gb = eng.cache_bytes() / 2**30
        s.rate, s.shared_frac, s.requests = wl.arrival_rate, wl.shared_frac, len(reqs)
        mc.finalize(s, wall)
        s.mean_batch = c["batch_size_sum"] / c["steps"] if c["steps"] else 0.0
        s.max_batch, s.preemptions, s.steps = c["max_running"], c["preemptions"], c["steps"]
        s.mean_step_ms = step_ms_sum / c["steps"] if c["steps"] else 0.0
        s.prefill_tokens, s.prefill_saved = c["prefill_tokens"], c["prefill_tokens_saved"]
        ps = eng.core.prefix_stats()
        q = ps["queried_blocks"] - ps0["queried_blocks"]
        s.prefix_hit_rate = (ps["hit_blocks"] - ps0["hit_blocks"]) / q if q else 0.0
        s.evictions = ps["evictions"] - ps0["evictions"]
        s.peak_kv_gb = s.peak_blocks * eng.bytes_per_block() / 2**30
        free_b, total_b = torch.cuda.mem_get_info()
        s.gpu_used_gb = (total_b - free_b) / 2**30
        print_summary(s)
        if summary_csv:
            append_bench_csv(summary_csv, s)
        return 0
    except Exception as e:  # noqa: BLE001
        print(f"error: {e}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
