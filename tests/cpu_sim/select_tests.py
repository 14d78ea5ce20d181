"""Writes tests/cpu_sim/selection.txt: the GPU tests that the CPU tier runs against the host build of the library.

    OPHIP_CPU_SIM_LIBRARY=$(python tests/cpu_sim/build_sim.py | tail -1) \\
        python -m pytest tests -m gpu -q -n 6 --timeout 300 --timeout-method signal --junitxml=/tmp/sim.xml
    python tests/cpu_sim/select_tests.py /tmp/sim.xml [seconds per test, default 2.5] [seconds per file, default 40]

Keeps every test that passed within the per-test limit, fastest first, until a file's share is used up; prints what
failed (tests that need the machine itself -- timings, the probe library, a C program linked against libophip.so -- do).
"""
import os
import sys
import xml.etree.ElementTree as ET

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    xml = sys.argv[1]
    per_test = float(sys.argv[2]) if len(sys.argv) > 2 else 2.5
    per_file = float(sys.argv[3]) if len(sys.argv) > 3 else 40.0
    files = {}
    failed = []
    for case in ET.parse(xml).getroot().iter("testcase"):
        path = case.get("classname").replace(".", "/") + ".py"
        node = "%s::%s" % (path, case.get("name"))
        if os.path.basename(path) in ("test_gpu_probe.py", "test_c_consumer.py"):  # they load libraries of their own, which need the machine
            continue
        if case.find("failure") is not None or case.find("error") is not None:
            failed.append(node)
        elif case.find("skipped") is None and float(case.get("time")) <= per_test:
            files.setdefault(path, []).append((float(case.get("time")), node))
    lines = ["# GPU tests that tests/test_cpu_sim_library.py runs against the host build (made by select_tests.py)"]
    total = 0
    for path in sorted(files):
        used = 0.0
        for t, node in sorted(files[path]):
            if used + t > per_file:
                break
            used += t
            lines.append(node)
        total += used
    open(os.path.join(HERE, "selection.txt"), "w").write("\n".join(lines) + "\n")
    print("%d tests selected, %.0f s of test time; %d failed:" % (len(lines) - 1, total, len(failed)))
    for f in failed:
        print("  " + f)


if __name__ == "__main__":
    main()
