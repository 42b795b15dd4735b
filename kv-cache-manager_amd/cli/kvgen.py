"""kvgen: from a model folder and prompts given as token ids to the generated ids, one line per prompt.

  kvgen --model DIR --prompt-ids 1,5,9 [--prompt-ids 4,4,2 ...] [--prompts-file FILE]
        [--max-new-tokens 16] [--temperature 0] [--sampler-seed 0] [--dump-tables]
        [engine flags of kvbench: --dtype --block-size --max-seq-len --num-blocks --pool-gb --max-num-seqs
         --max-batched-tokens --prefill-chunk --prefix --policy --attn --eos-id --no-graphs --no-programs]
  kvgen --random-weights --sizes tiny-a ...      (random weights instead of a folder, as the other tools take them)

--prompt-ids may be given several times ("--prompt-ids=1,2 --prompt-ids=3"); --prompts-file holds one prompt a
line, ids separated by commas or blanks.  The prompts run together through the scheduler (add / step /
take_finished, as the reference's correctness tool generates: src/main_correct.cpp:61-80).  Standard output
gets one line of blank-separated generated ids per prompt, in the order the prompts were given (an empty line
for a prompt that can never fit the cache pool).  --dump-tables: after every step, one line on standard error
with the step's number and the live requests' page tables.
"""
import json
import sys

from .args import Args
from .common import engine_config_from_args, make_engine


def _ids(text):
    return [int(t) for t in text.replace(",", " ").split()]


def main(argv=None):
    argv = list(sys.argv[1:] if argv is None else argv)
    try:
        # --prompt-ids may repeat: Args keeps one value per flag, so they are taken out first
        prompts, rest, i = [], [], 0
        while i < len(argv):
            arg = argv[i]
            if arg.startswith("--prompt-ids="):
                prompts.append(_ids(arg.split("=", 1)[1]))
            elif arg == "--prompt-ids":
                if i + 1 >= len(argv):
                    raise ValueError("--prompt-ids needs a list of ids")
                i += 1
                prompts.append(_ids(argv[i]))
            else:
                rest.append(arg)
            i += 1
        a = Args(rest)
        if a.has("prompts-file"):
            with open(a.str("prompts-file", "")) as f:
                prompts += [_ids(line) for line in f if line.strip()]
        if not prompts or any(not p for p in prompts):
            raise ValueError("give at least one prompt: --prompt-ids 1,5,9 (may repeat) or --prompts-file FILE")
        new, temperature, seed = a.i32("max-new-tokens", 16), a.f64("temperature", 0.0), a.i64("sampler-seed", 0)
        if new <= 0:
            raise ValueError("--max-new-tokens must be positive")
        dump = a.flag("dump-tables")
        ec = engine_config_from_args(a)
        eng = make_engine(a, ec)
        a.warn_unused()
        ids = [eng.add_request(p, new, temperature, seed) for p in prompts]
        done, step = {}, 0
        while not eng.idle():
            eng.step()
            if dump:
                tables = {}
                for k, rid in enumerate(ids):
                    if rid in done:
                        continue
                    groups = [eng.core.seq_table(rid, g) for g in range(eng.core.num_groups)]
                    if any(groups):
                        tables[k] = groups
                print(json.dumps({"step": step, "tables": tables}), file=sys.stderr, flush=True)
            for f in eng.take_finished():
                done[f.id] = f.generated
            step += 1
        for rid in ids:
            print(" ".join(str(t) for t in done.get(rid, [])), flush=True)
        return 0
    except Exception as e:                                       # a tool: one line, exit code 1
        print(f"kvgen: {e}", file=sys.stderr)
        return 1
