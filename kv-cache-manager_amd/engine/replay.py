"""Trace replay: given token ids are fed through the model step by step and logits are written
out.  Nothing is sampled.  It drives the same model, step function, cache manager and kernels
that generation uses.  The nearest thing in the reference is Engine::score, which scores one
whole sequence in one step through the real manager (src/engine/engine.cpp:92-108).

A step is a JSON object  {"step": k, "entries": [{"id": .., "tokens": [..], "want": [..]}], "end": [..]}:
all entries are one batch; a request's tokens continue where its last entry stopped; ``want``
are places among this entry's tokens whose logits are asked for; ``end`` lists requests whose
pages are given back after the step.
"""
import json
import os
import sys

import numpy as np

from ..config.engine_config import EngineConfig
from .build import build_runner


class ReplayError(RuntimeError):
    pass


class TraceReplayer:
    def __init__(self, model_dir, dtype="bfloat16", max_tokens=4096, block_size=16, device="cuda:0",
                 max_live=8, attn="auto", architecture=None, model_config=None, tensors=None, use_programs=False,
                 fold_norms=True):
        """``model_dir``: a model folder; or None with architecture + model_config + tensors (checkpoint
        names -> tensors in memory), as build_runner takes them.  ``use_programs``: steps run as generation
        runs them by default, from launch lists recorded once per step shape (a step's rows and wanted rows
        padded to multiples of 64) and replayed with only the step's metadata changed; a model with a part
        that is not capturable, and steps that want more rows than one head launch takes, run launch by
        launch all the same."""
        pages = (max_tokens + block_size - 1) // block_size
        span = max(pages * block_size, block_size)
        ec = EngineConfig(policy="paged", block_size=block_size, max_seq_len=span, num_blocks=max(pages, 1),
                          watermark_blocks=0, max_num_seqs=max_live, max_batched_tokens=span,
                          max_logit_rows=min(-(-span // 64) * 64, 1024), dtype=dtype, attn=attn, use_graphs=False,
                          fold_norms=fold_norms, beyond_max_position=True)     # a trace's lengths are given, not generated
        self.runner, self.core, self.model, self.model_config = build_runner(
            model_dir, ec, device=device, architecture=architecture, model_config=model_config, tensors=tensors)
        self.vocab_size = self.model.spec.vocab_size
        self._ids = {}          # external id -> integer id
        self._next = 0
        self._computed = {}     # integer id -> tokens already run
        self.programs = {} if (use_programs and self.model.capturable) else None      # StepShape -> ops.StepProgram
        self.steps_replayed = 0

    # -------------------------------------------------------------------- recorded step shapes
    def _shape_of(self, entries):
        """The shape a step of these entries is recorded and replayed in, or None when it takes the
        direct path (more wanted rows, or more rows, than the buffers of one launch hold)."""
        from .graphs import StepShape
        lim = self.runner.limits
        rows = sum(e[2] for e in entries)
        wanted = sum(len(e[3]) for e in entries)
        leading = 0
        while leading < len(entries) and entries[leading][2] == 1:
            leading += 1
        run = max(e[2] for e in entries)
        shape = StepShape(rows=-(-rows // 64) * 64, seqs=len(entries), leading=leading, logit_rows=-(-wanted // 64) * 64,
                          max_run=1 if run == 1 else -(-run // 64) * 64, context_bound=lim.max_context_len,
                          table_stride=lim.max_blocks_per_seq)
        if wanted == 0 or shape.rows > lim.max_tokens or shape.logit_rows > lim.max_logit_rows:
            return None
        return shape

    def _run_recorded(self, entries, shape):
        """One step in its recorded shape: the first of a shape runs through the parts while its launches
        are recorded, later ones replay the list.  -> float32 logits [wanted, vocab] on the host."""
        import torch
        from .graphs import RecordedStepContext
        runner, ops = self.runner, self.runner.ops
        layout = self.core.build_batch(entries, runner.host_buffer(), pad_rows=shape.rows, pad_seqs=shape.seqs,
                                       pad_logit_rows=shape.logit_rows, table_stride=shape.table_stride)
        runner._check(layout)
        runner.upload(layout)
        program = self.programs.get(shape)
        if program is None:
            step = RecordedStepContext(runner, layout, shape)
            program = ops.StepProgram()
            with ops.recording(program):
                logits = runner.model.forward(step)
            self.programs[shape] = program
        else:
            program.run()
            self.steps_replayed += 1
            logits = runner.workspace.get("logits", (shape.logit_rows, self.vocab_size), torch.float32)
        return logits[:layout.logit_rows].cpu().numpy()

    def tables(self):
        """Page tables of the live requests, per cache group: {request: [[page ids of group 0], ...]}
        (-1: a page a window has passed and given back)."""
        return {json.loads(key): [self.core.seq_table(sid, g) for g in range(self.core.num_groups)]
                for key, sid in self._ids.items()}

    def _sid(self, ext, create):
        key = json.dumps(ext)
        if key not in self._ids:
            if not create:
                raise ReplayError(f"request {ext!r} is not live")
            self._ids[key] = self._next
            self._next += 1
        return self._ids[key]

    def step(self, record):
        """Runs one step; returns float32 logits [wanted, vocab] or None when nothing is wanted."""
        entries, seen = [], set()
        for e in record.get("entries", []):
            tokens = [int(t) for t in e["tokens"]]
            want = [int(w) for w in e.get("want", [])]
            if not tokens:
                raise ReplayError(f"request {e['id']!r}: an entry needs at least one token")
            if any(t < 0 or t >= self.vocab_size for t in tokens):
                raise ReplayError(f"request {e['id']!r}: token id outside the vocabulary of {self.vocab_size}")
            if any(w < 0 or w >= len(tokens) for w in want):
                raise ReplayError(f"request {e['id']!r}: a wanted place lies outside its {len(tokens)} tokens")
            fresh = json.dumps(e["id"]) not in self._ids
            sid = self._sid(e["id"], create=True)
            if sid in seen:
                raise ReplayError(f"request {e['id']!r} appears twice in one step")
            seen.add(sid)
            if fresh:
                self.core.seq_new(sid, tokens)
                if not self.core.can_admit(sid):
                    self.core.seq_delete(sid)
                    del self._ids[json.dumps(e["id"])]
                    raise ReplayError(f"request {e['id']!r} does not fit the cache pool (--max-tokens is too small)")
                self.core.admit(sid)
                self._computed[sid] = 0
            else:
                self.core.seq_push_tokens(sid, tokens)
                if not self.core.append_slot(sid):
                    raise ReplayError(f"out of cache pages while extending request {e['id']!r} (--max-tokens is too small)")
            entries.append((sid, self._computed[sid], len(tokens), want))
        logits = None
        if entries:
            shape = self._shape_of(entries) if self.programs is not None else None
            if shape is not None:
                logits = self._run_recorded(entries, shape)
            else:
                layout = self.core.build_batch(entries, self.runner.host_buffer())
                logits = self.runner.execute_to_host(layout)
            for sid, start, count, _ in entries:
                self._computed[sid] = start + count
                self.core.set_computed(sid, start + count)
                self.core.commit(sid)
        for ext in record.get("end", []):
            sid = self._sid(ext, create=False)
            self.core.release(sid)
            self.core.seq_delete(sid)
            del self._ids[json.dumps(ext)]
            del self._computed[sid]
        return logits


def scheduled_replay(engine, requests, arrivals=None, max_steps=1 << 20, on_step=None):
    """The second way to replay given tokens: through the engine's own scheduler.  Each request is
    (prompt tokens, continuation tokens): it is admitted, cut into portions, preempted and served
    from prefix hits as the engine's options decide, and wherever a token would be sampled the next
    token of the continuation is pushed instead (the sampled id is ignored).  Returns, per request in
    order, the logits those tokens were to be sampled from: [len(continuation), vocab], i.e. the
    logits at positions len(prompt) - 1 .. len(prompt) + len(continuation) - 2 of the whole sequence.
    The reference scores given tokens one whole sequence at a time (src/main_correct.cpp:194-222)
    and generates through add/step/take_finished (main_correct.cpp:61-80); this does both at once.

    arrivals[i]: the step before which request i is added (default: all before the first step).
    on_step(step number, StepInfo, {request index: engine id}): called after every step."""
    arrivals = list(arrivals) if arrivals is not None else [0] * len(requests)
    order = sorted(range(len(requests)), key=lambda i: (arrivals[i], i))
    ids, nxt, steps = {}, 0, 0
    while nxt < len(order) or not engine.idle():
        while nxt < len(order) and arrivals[order[nxt]] <= steps:
            i = order[nxt]
            prompt, continuation = requests[i]
            ids[i] = engine.add_request(prompt, len(continuation), forced=continuation)
            nxt += 1
        info = engine.step()
        if on_step is not None:
            on_step(steps, info, ids)
        engine.take_finished()
        steps += 1
        if steps > max_steps:
            raise ReplayError("scheduled_replay: the engine does not come to an end")
    return [engine.forced_logits(ids[i]) for i in range(len(requests))]


def _write_tables(out_dir, step, tables):
    with open(os.path.join(out_dir, f"{step}.tables.json"), "w") as f:
        json.dump({"step": step, "tables": [{"id": k, "groups": v} for k, v in tables.items()]}, f)


def main(argv=None):
    argv = list(sys.argv[1:] if argv is None else argv)
    if "--scheduled" in argv:
        return scheduled_main(argv)
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description="replay given token ids step by step and write logits "
                                 "(--scheduled: through the engine's own scheduler, one request per input line)")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--attn", default="auto", choices=["v1", "v2", "auto"])
    ap.add_argument("--recorded", action="store_true",
                    help="run steps as generation does by default: from launch lists recorded once per step shape")
    ap.add_argument("--dump-tables", action="store_true",
                    help="also write <step>.tables.json: the live requests' page tables after the step, per cache group")
    args = ap.parse_args(argv)
    os.makedirs(args.out, exist_ok=True)
    print(f"[trace_run] loading {args.model} ({args.dtype})", file=sys.stderr, flush=True)
    rp = TraceReplayer(args.model, args.dtype, args.max_tokens, args.block_size, attn=args.attn, use_programs=args.recorded)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    for number, line in enumerate(sys.stdin, 1):
        line = line.strip()
        if not line:
            continue
        try:
            record = json.loads(line)
            if not isinstance(record, dict) or "step" not in record:
                raise ReplayError('a step is a JSON object {"step": .., "entries": [..], "end": [..]}')
            if args.dump_tables:      # before the step's ``end`` gives the pages back
                ended, record = record.get("end", []), dict(record, end=[])
                logits = rp.step(record)
                _write_tables(args.out, record["step"], rp.tables())
                rp.step({"step": record["step"], "entries": [], "end": ended})
            else:
                logits = rp.step(record)
        except (ReplayError, ValueError, KeyError, TypeError) as e:      # what the input can get wrong: one line, exit 1
            what = f"missing key {e}" if isinstance(e, KeyError) else str(e)
            print(f"trace_run: input line {number}: {what}", file=sys.stderr, flush=True)
            return 1
        if logits is not None:
            np.ascontiguousarray(logits, dtype="<f4").tofile(os.path.join(args.out, f"{record['step']}.f32"))
        print(f"done {record['step']}", flush=True)
    return 0


def scheduled_main(argv):
    """trace_run --scheduled: the second way to replay given tokens.  Standard input holds one request a
    line, {"id": .., "prompt": [..], "forced": [..], "arrival": k}: the request joins before step k
    (default 0) and goes through the engine's own scheduler under the engine flags the serving tools
    take (--block-size, --num-blocks | --pool-gb, --max-seq-len, --max-num-seqs, --max-batched-tokens,
    --prefill-chunk, --prefix, --watermark, --policy, --attn, --no-graphs, --no-programs, --no-fold-norms);
    every token it would sample is replaced by the next of ``forced``.  <id>.f32 in --out receives the
    logits those tokens were to be sampled from, [len(forced), vocab] little-endian 32-bit floats, and
    ``done <id>`` is printed per request.  --dump-tables writes <step>.tables.json after every step.
    The reference's pieces of this: generation through add / step / take_finished
    (src/main_correct.cpp:61-80) and teacher-forced scoring of given tokens (main_correct.cpp:194-222)."""
    from ..cli.args import Args
    from ..cli.common import engine_config_from_args
    from .engine import Engine
    try:
        a = Args([x for x in argv if x != "--scheduled"])
        model, out = a.str("model", ""), a.str("out", "")
        if not model or not out:
            raise ValueError("give --model DIR and --out DIR")
        dtype = a.str("dtype", "bfloat16")
        dump = a.flag("dump-tables")
        ec = engine_config_from_args(a, dtype=dtype, beyond_max_position=True)       # a trace's lengths are given
        a.warn_unused()
    except ValueError as e:
        print(f"trace_run: {e}", file=sys.stderr, flush=True)
        return 2
    os.makedirs(out, exist_ok=True)
    requests, names, arrivals = [], [], []
    for number, line in enumerate(sys.stdin, 1):
        line = line.strip()
        if not line:
            continue
        try:
            r = json.loads(line)
            if not isinstance(r, dict):
                raise ReplayError('a request is a JSON object {"id": .., "prompt": [..], "forced": [..], "arrival": k}')
            prompt, forced = [int(t) for t in r["prompt"]], [int(t) for t in r["forced"]]
            if not prompt or not forced:
                raise ReplayError(f"request {r['id']!r}: prompt and forced need at least one token each")
            if not isinstance(r["id"], (str, int)) or isinstance(r["id"], bool) or any(c in str(r["id"]) for c in "/\\\0") \
                    or str(r["id"]) in ("", ".", ".."):
                raise ReplayError(f"request id {r['id']!r} must be a number or a string that can name a file (<id>.f32)")
            if str(r["id"]) in {str(n) for n in names}:
                raise ReplayError(f"request {r['id']!r} appears twice")
            names.append(r["id"])
            requests.append((prompt, forced))
            arrivals.append(int(r.get("arrival", 0)))
        except (ReplayError, ValueError, KeyError, TypeError) as e:
            what = f"missing key {e}" if isinstance(e, KeyError) else str(e)
            print(f"trace_run: input line {number}: {what}", file=sys.stderr, flush=True)
            return 1
    print(f"[trace_run] loading {model} ({dtype}); {len(requests)} requests through the scheduler", file=sys.stderr, flush=True)
    eng = Engine(model, ec)
    print("[trace_run] ready", file=sys.stderr, flush=True)

    def after_step(step, info, ids):
        if dump:
            live = {}
            for i, rid in ids.items():
                try:
                    groups = [eng.core.seq_table(rid, g) for g in range(eng.core.num_groups)]
                except Exception:        # finished and collected already
                    continue
                if any(groups):          # a waiting or finished request holds no page
                    live[json.dumps(names[i])] = groups
            _write_tables(out, step, {json.loads(k): v for k, v in live.items()})

    try:
        logits = scheduled_replay(eng, requests, arrivals, on_step=after_step)
    except (ReplayError, ValueError) as e:
        print(f"trace_run: {e}", file=sys.stderr, flush=True)
        return 1
    for name, rows in zip(names, logits):
        np.ascontiguousarray(rows, dtype="<f4").tofile(os.path.join(out, f"{name}.f32"))
        print(f"done {name}", flush=True)
    k = eng.core.counters()
    print(f"[trace_run] {k['steps']} steps, {k['preemptions']} preemptions, {k['rejected']} rejected, "
          f"{k['prefill_tokens_saved']} prompt tokens served from the prefix cache", file=sys.stderr, flush=True)
    return 0
