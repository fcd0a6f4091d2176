"""Read-only board telemetry from sysfs: no child process, so it is safe to call from a process
that already uses the GPU (and under a profiler)."""
import glob
import re


def sclk_mhz():
    """Current shader clock in MHz: the level marked `*` in pp_dpm_sclk of the first card, or None."""
    for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
        try:
            with open(path) as f:
                for line in f:
                    m = re.match(r"\s*\d+:\s*(\d+)\s*Mhz\s*\*", line, re.IGNORECASE)
                    if m:
                        return int(m.group(1))
        except OSError:
            continue
    return None


def power_w():
    """Current package power in watts (hwmon power1_input, microwatts), or None."""
    for path in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")):
        try:
            with open(path) as f:
                return int(f.read().strip()) / 1e6
        except (OSError, ValueError):
            continue
    return None
