"""The summaries of rocprofv3 runs that the profiles are made with, on small files written here."""
import csv

from fllm_amd.kernels.trace_summary import summarize, summarize_counters


def test_kernel_time_of_the_last_steps(tmp_path):
    path = tmp_path / "1_kernel_trace.csv"
    with open(path, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["Kernel_Name", "Start_Timestamp", "End_Timestamp"])
        t = 0
        for step in range(4):
            for name, us in (("embed_kernel", 2), ("product", 10 * (step + 1)), ("product", 10 * (step + 1))):
                w.writerow([name, t, t + us * 1000])
                t += us * 1000 + 1000
    lines = summarize(str(tmp_path), steps=2, top=5)
    # steps 1 and 2 are added up (the last start only closes the span): products of 20 and 30 us, two a step
    assert lines[0].startswith("2 steps: 55.0 us a step")
    assert lines[2].split()[:3] == ["50.0", "2.0", "25.00"]


def test_counters_a_dispatch(tmp_path):
    path = tmp_path / "7_counter_collection.csv"
    with open(path, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value"])
        for d in range(1, 7):
            name = "a" if d % 2 else "b"
            w.writerow([d, name, "SQ_WAVES", 100 * d])
            w.writerow([d, name, "SQ_WAVES", 1])        # a counter may come in several rows of one dispatch: they add
            w.writerow([d, name, "TCC_HIT_sum", d])
    lines = summarize_counters(str(tmp_path), last=4)
    text = "\n".join(lines)
    assert "last 4 dispatches" in lines[0]
    # dispatches 3..6: a has 3 and 5, b has 4 and 6
    at = lines.index("a  (2 dispatches)")
    assert lines[at + 1].split() == ["SQ_WAVES", "401.0"] and lines[at + 2].split() == ["TCC_HIT_sum", "4.0"]
    at = lines.index("b  (2 dispatches)")
    assert lines[at + 1].split() == ["SQ_WAVES", "501.0"], text
