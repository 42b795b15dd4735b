"""``--key=value`` / ``--key value`` / ``--flag`` command lines with typed getters, defaults and
a warning for flags nobody read, as the reference's tools parse theirs (src/common/args.h:12-58)."""
import sys


class Args:
    def __init__(self, argv):
        self.kv, self.used = {}, set()
        i = 0
        while i < len(argv):
            a = argv[i]
            if not a.startswith("--"):
                raise ValueError(f"bad argument: {a}")
            a = a[2:]
            if "=" in a:
                k, v = a.split("=", 1)
                self.kv[k] = v
            elif i + 1 < len(argv) and not argv[i + 1].startswith("--"):
                i += 1
                self.kv[a] = argv[i]
            else:
                self.kv[a] = "1"
            i += 1

    def has(self, k):
        self.used.add(k)
        return k in self.kv

    def str(self, k, default):
        self.used.add(k)
        return self.kv.get(k, default)

    def i64(self, k, default):
        s = self.str(k, "")
        return int(s) if s != "" else default

    i32 = i64

    def f64(self, k, default):
        s = self.str(k, "")
        return float(s) if s != "" else default

    def flag(self, k, default=False):
        s = self.str(k, "")
        return default if s == "" else s in ("1", "true", "on", "yes")

    def warn_unused(self):
        for k in sorted(self.kv):
            if k not in self.used:
                print(f"warning: unused flag --{k}", file=sys.stderr)
