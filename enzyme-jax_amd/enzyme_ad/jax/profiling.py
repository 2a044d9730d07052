"""Timing in the style of the reference's test/xprof_utils.py:62-150
(`profile_compiled_function`): run N times, report the minimum step time.
Device time comes from HIP events recorded on the stream the work runs on."""
import torch


def profile_compiled_function(fn, args=(), nrepeat=5, warmup=1):
    """Returns (min_seconds, all_seconds) over `nrepeat` timed calls."""
    stream = torch.cuda.current_stream()
    for _ in range(warmup):
        fn(*args)
    stream.synchronize()
    times = []
    for _ in range(nrepeat):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        fn(*args)
        e1.record(stream)
        e1.synchronize()
        times.append(e0.elapsed_time(e1) * 1e-3)
    return min(times), times


def pretty_print_table(name, pname, backend, key, time):
    """One result line, columns as test/test_utils.py:589-596."""
    line = "{:<20}\t{:<20}\t{:<15}\t{:<10}\t{:<15.8f}".format(name, pname, backend, key, time)
    print(line, flush=True)
    return "{}\t{}\t{}\t{}\t{}".format(name, pname, backend, key, time)


CSV_HEADER = ["Benchmark Name", "Pass Pipeline", "Backend", "Key", "Time"]   # test/test_utils.py:609-611
