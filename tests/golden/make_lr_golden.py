"""Writes tests/golden/lr_schedule.json: learning rates (FP32 bit patterns) produced by the
reference's own LRScheduler (include/training/lr_scheduler.h), through oracle/_ref/lr_dump_ref,
which `make -C oracle ref` compiles from oracle/lr_dump.cpp and the reference's header.
Run in the build container, where /root/reference exists."""
import json
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))

if __name__ == "__main__":
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-s", "ref"], check=True)
    out = subprocess.run([os.path.join(ROOT, "oracle", "_ref", "lr_dump_ref")], check=True, capture_output=True,
                         text=True).stdout
    data = json.loads(out)
    with open(os.path.join(HERE, "lr_schedule.json"), "w") as f:
        json.dump(data, f, separators=(",", ":"))
        f.write("\n")
    print({k: len(v) for k, v in data.items()})
