"""Writes tests/golden/schedule_vectors.json: `PipeSchedParams.rank_works` of the
REFERENCE (pfeife/schedule/scheduler.py, a file with no third-party imports) for
a grid of (device_cnt, batch_cnt, node_cnt, loop_batch, prefetch_fwd).

Run in the build container only (the reference does not travel):
    python tests/golden/make_schedule_vectors.py
"""
import importlib.util
import json
import os

REF = "/root/reference/pfeife/schedule/scheduler.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "schedule_vectors.json")


def main():
    spec = importlib.util.spec_from_file_location("ref_scheduler", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    cases = []
    for device_cnt in (1, 2, 3, 4):
        for node_cnt in (1, 2, 3, 4, 8):
            if node_cnt < device_cnt:
                continue
            for batch_cnt in (1, 2, 4, 6, 8):
                for loop_batch in sorted({1, 2, device_cnt, batch_cnt}):
                    if loop_batch > batch_cnt:
                        continue
                    for prefetch_fwd in (0, 1):
                        try:
                            p = mod.PipeSchedParams(device_cnt, batch_cnt, node_cnt, loop_batch, prefetch_fwd)
                        except Exception as e:  # the reference itself rejects / breaks on this tuple
                            cases.append(dict(args=[device_cnt, batch_cnt, node_cnt, loop_batch, prefetch_fwd],
                                              error=type(e).__name__))
                            continue
                        cases.append(dict(args=[device_cnt, batch_cnt, node_cnt, loop_batch, prefetch_fwd],
                                          rank_works=[[[n, b, int(f)] for n, b, f in w] for w in p.rank_works]))
    with open(OUT, "w") as f:
        json.dump(cases, f, separators=(",", ":"))
    print("wrote %d cases to %s" % (len(cases), OUT))


if __name__ == "__main__":
    main()
