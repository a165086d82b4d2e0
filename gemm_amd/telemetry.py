"""Socket power and shader clock of the GPU while something else runs: a host thread that polls amdsmi.

The measurements of this repository say that a GEMM on random data is bound by the chip's power limit, not by its
matrix cores' issue rate; this module puts the observation beside the inference: `Sampler` reads the board's own
telemetry (socket power, the shader clock of every XCD, the hot-spot temperature) every few milliseconds from a
host thread, makes no HIP call and starts no process, so it can run around child processes as well as around
launches of this process.  Samples carry `time.monotonic()` stamps, the clock a child's CLOCK_MONOTONIC stamps share.

Where amdsmi is missing or refuses, `Sampler` stays empty and `summary()` says why: telemetry never fails a run.
"""
import threading
import time


class Sampler:
    def __init__(self, period_s=0.004, device_index=0):
        self.period_s = period_s
        self.samples = []   # (monotonic seconds, socket power W, mean shader clock MHz, min over XCDs, max over XCDs, hot spot C)
        self.error = None
        self.power_limit_w = None
        self._stop = threading.Event()
        self._thread = None
        self._smi = None
        self._handle = None
        try:
            import amdsmi
            amdsmi.amdsmi_init()
            handles = amdsmi.amdsmi_get_processor_handles()
            if not handles:
                raise RuntimeError("amdsmi reports no GPU")
            self._smi, self._handle = amdsmi, handles[min(device_index, len(handles) - 1)]
            try:
                cap = amdsmi.amdsmi_get_power_cap_info(self._handle).get("power_cap")
                self.power_limit_w = float(cap) / 1e6 if isinstance(cap, (int, float)) and cap > 0 else None
            except Exception:   # the cap is a nicety
                pass
        except Exception as e:   # ImportError, AmdSmiLibraryException, missing driver files ...
            self.error = f"{type(e).__name__}: {e}"

    @staticmethod
    def _num(x):
        return float(x) if isinstance(x, (int, float)) else None

    def _poll(self):
        m = self._smi.amdsmi_get_gpu_metrics_info(self._handle)
        clks = [c for c in (m.get("current_gfxclks") or []) if isinstance(c, (int, float))]
        if not clks and isinstance(m.get("current_gfxclk"), (int, float)):
            clks = [m["current_gfxclk"]]
        return (time.monotonic(), self._num(m.get("current_socket_power")),
                sum(clks) / len(clks) if clks else None, min(clks) if clks else None, max(clks) if clks else None,
                self._num(m.get("temperature_hotspot")))

    def _run(self):
        while not self._stop.is_set():
            try:
                self.samples.append(self._poll())
            except Exception as e:
                self.error = f"{type(e).__name__}: {e}"
                return
            self._stop.wait(self.period_s)

    def start(self):
        if self._smi is not None and self._thread is None:
            self._stop.clear()
            self._thread = threading.Thread(target=self._run, name="neogemm-telemetry", daemon=True)
            self._thread.start()
        return self

    def stop(self):
        if self._thread is not None:
            self._stop.set()
            self._thread.join()
            self._thread = None
        return self

    def __enter__(self):
        return self.start()

    def __exit__(self, *exc):
        self.stop()
        return False

    def summary(self, t0=None, t1=None):
        """Mean / extremes over the samples taken in [t0, t1] (monotonic seconds; None: no bound)."""
        if self._smi is None:
            return {"available": False, "error": self.error}
        rows = [s for s in self.samples if (t0 is None or s[0] >= t0) and (t1 is None or s[0] <= t1)]
        out = {"available": True, "source": "amdsmi gpu_metrics, host thread", "samples": len(rows),
               "period_ms": round(self.period_s * 1e3, 2), "power_limit_w": self.power_limit_w}
        if self.error:
            out["error"] = self.error

        def stats(idx, name, lo_idx=None, hi_idx=None):
            vals = [r[idx] for r in rows if r[idx] is not None]
            if not vals:
                return
            out[name] = {"mean": round(sum(vals) / len(vals), 1),
                         "min": round(min(r[lo_idx or idx] for r in rows if r[lo_idx or idx] is not None), 1),
                         "max": round(max(r[hi_idx or idx] for r in rows if r[hi_idx or idx] is not None), 1)}

        stats(1, "socket_power_w")
        stats(2, "shader_clock_mhz", 3, 4)   # mean over XCDs and samples; min / max over single XCDs
        stats(5, "hotspot_c")
        return out
