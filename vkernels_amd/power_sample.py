"""Socket power and shader clock of the GPU while a command runs.

    python -m vkernels_amd.power_sample [--hz 20] [--smi-every 1.0] -- <command ...>

Starts the command as a child process and, until it ends, reads what the amdgpu driver
publishes for card 0 under /sys/class/drm: `power1_input` (socket power, microwatts) and
`power1_cap` of its hwmon directory, and the level that `pp_dpm_sclk` marks as current
(MHz).  Once per --smi-every seconds it also asks `amd-smi metric --power --clock --json`
for the shader clock of every XCD.  Prints the command's output as it comes and then one
JSON line: mean / max of the samples taken while the GPU was busy (power above the idle
floor by more than 20 %), next to the cap.  Nothing here touches a GPU setting.
"""
from __future__ import annotations

import argparse
import glob
import json
import re
import statistics
import subprocess
import sys
import threading
import time


def _read(path: str) -> str | None:
    try:
        with open(path) as fh:
            return fh.read()
    except OSError:
        return None


def _sclk_mhz(text: str | None) -> float | None:
    """The level of pp_dpm_sclk marked with a star."""
    if not text:
        return None
    for line in text.splitlines():
        if line.rstrip().endswith("*"):
            m = re.search(r"(\d+)\s*Mhz", line, re.I)
            if m:
                return float(m.group(1))
    return None


def _smi_clocks() -> list[float]:
    try:
        res = subprocess.run(["amd-smi", "metric", "-g", "0", "--power", "--clock", "--json"],
                             capture_output=True, text=True, timeout=10)
        data = json.loads(res.stdout)
    except (OSError, ValueError, subprocess.SubprocessError):
        return []
    gpu = data.get("gpu_data", data if isinstance(data, list) else [data])[0]
    clocks = []
    for name, rec in (gpu.get("clock") or {}).items():
        if name.startswith("gfx") and isinstance(rec, dict):
            v = (rec.get("clk") or {}).get("value") if isinstance(rec.get("clk"), dict) else rec.get("clk")
            if isinstance(v, (int, float)):
                clocks.append(float(v))
    return clocks


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--hz", type=float, default=20.0)
    ap.add_argument("--smi-every", type=float, default=1.0, help="seconds between amd-smi readings (0 = none)")
    ap.add_argument("command", nargs=argparse.REMAINDER)
    args = ap.parse_args()
    cmd = args.command[1:] if args.command[:1] == ["--"] else args.command
    if not cmd:
        ap.error("no command given")

    hwmon = sorted(glob.glob("/sys/class/drm/card0/device/hwmon/hwmon*"))
    power_path = hwmon[0] + "/power1_input" if hwmon else None
    cap = _read(hwmon[0] + "/power1_cap") if hwmon else None
    sclk_path = "/sys/class/drm/card0/device/pp_dpm_sclk"
    samples: list[tuple[float, float | None, float | None]] = []   # time, watts, MHz
    smi: list[tuple[float, list[float]]] = []
    done = threading.Event()

    def sample_sysfs():
        period = 1.0 / args.hz
        while not done.is_set():
            t = time.monotonic()
            p = _read(power_path) if power_path else None
            watts = float(p) / 1e6 if p and p.strip().isdigit() else None
            samples.append((t, watts, _sclk_mhz(_read(sclk_path))))
            done.wait(max(0.0, period - (time.monotonic() - t)))

    def sample_smi():
        while not done.is_set():
            t = time.monotonic()
            c = _smi_clocks()
            if c:
                smi.append((t, c))
            done.wait(max(0.0, args.smi_every - (time.monotonic() - t)))

    threads = [threading.Thread(target=sample_sysfs, daemon=True)]
    if args.smi_every > 0:
        threads.append(threading.Thread(target=sample_smi, daemon=True))
    idle = _read(power_path) if power_path else None
    for th in threads:
        th.start()
    t0 = time.monotonic()
    rc = subprocess.call(cmd)
    done.set()
    for th in threads:
        th.join(timeout=15)

    watts = [w for _, w, _ in samples if w is not None]
    idle_w = float(idle) / 1e6 if idle and idle.strip().isdigit() else (min(watts) if watts else None)
    floor = min(watts) if watts else None
    busy = [(w, f) for _, w, f in samples if w is not None and floor is not None and w > 1.2 * floor]
    busy_t = [t for t, w, _ in samples if w is not None and floor is not None and w > 1.2 * floor]
    smi_busy = [c for t, c in smi if busy_t and busy_t[0] <= t <= busy_t[-1]]

    def stats(values):
        values = [v for v in values if v is not None]
        if not values:
            return None
        return {"mean": round(statistics.mean(values), 1), "median": round(statistics.median(values), 1),
                "min": round(min(values), 1), "max": round(max(values), 1), "n": len(values)}

    out = {
        "command": cmd, "rc": rc, "seconds": round(time.monotonic() - t0, 2), "hz": args.hz,
        "samples": len(samples),
        "power_cap_w": float(cap) / 1e6 if cap and cap.strip().isdigit() else None,
        "idle_power_w": idle_w,
        "busy_power_w": stats([w for w, _ in busy]),
        "busy_sclk_mhz_sysfs": stats([f for _, f in busy]),
        "busy_sclk_mhz_amd_smi_per_xcd": stats([v for c in smi_busy for v in c]),
        "busy_sclk_mhz_amd_smi_slowest_xcd": stats([min(c) for c in smi_busy]),
        "amd_smi_readings": len(smi_busy),
    }
    print(json.dumps(out))
    return rc


if __name__ == "__main__":
    sys.exit(main())
