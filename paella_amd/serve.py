"""ctypes front-end of include/paella_serve.h: run the llis server and the load generator inside this process."""
import ctypes
import os

from . import _abi

MAX_TYPES = 16
c_int, c_uint, c_float, c_double, c_char_p, c_void_p, c_size_t = (ctypes.c_int, ctypes.c_uint, ctypes.c_float, ctypes.c_double,
                                                                  ctypes.c_char_p, ctypes.c_void_p, ctypes.c_size_t)


class ServerOptions(ctypes.Structure):
    _fields_ = [("name", c_char_p), ("sched", c_char_p), ("num_streams", c_uint), ("extra_kernels", c_uint), ("unfair", c_float),
                ("sched_sleep", c_uint), ("mem_marker", c_int), ("event_log", c_int), ("cpu", c_int), ("measure_block_time", c_int), ("noti_batch", c_uint), ("print_ipc_latency", c_int),
                ("placement", c_int)]


class LoadOptions(ctypes.Structure):
    _fields_ = [("server_name", c_char_p), ("num_types", c_int), ("job_paths", c_char_p * MAX_TYPES), ("proportions", c_float * MAX_TYPES),
                ("max_outstanding", c_uint * MAX_TYPES), ("iat_us", c_double), ("dist_exp", c_int), ("ln_sigma", c_double),
                ("concurrency", c_int), ("num_jobs", c_uint), ("warmup_jobs", c_uint), ("seed", c_uint), ("pin_threads", c_int),
                ("profile_prefix", c_char_p), ("trace_path", c_char_p), ("verify", c_int), ("verify_expected", c_void_p),
                ("verify_expected_bytes", c_size_t)]


class LatencyStats(ctypes.Structure):
    _fields_ = [("mean", c_double), ("p50", c_double), ("p90", c_double), ("p95", c_double), ("p99", c_double), ("max", c_double),
                ("sd", c_double), ("count", ctypes.c_uint64)]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_}


class LoadResult(ctypes.Structure):
    _fields_ = [("elapsed_us", c_double), ("throughput_rps", c_double), ("all", LatencyStats), ("per_type", LatencyStats * MAX_TYPES),
                ("queue_full_events", c_uint), ("type_full_events", c_uint), ("verified_requests", ctypes.c_uint64), ("mismatches", ctypes.c_uint64)]


class DirectOptions(ctypes.Structure):
    _fields_ = [("num_types", c_int), ("models", c_char_p * MAX_TYPES), ("proportions", c_float * MAX_TYPES),
                ("max_outstanding", c_uint * MAX_TYPES), ("seed_weights", ctypes.c_uint64), ("num_streams", c_int), ("iat_us", c_double),
                ("dist_exp", c_int), ("ln_sigma", c_double), ("num_jobs", c_uint), ("warmup_jobs", c_uint), ("seed", c_uint),
                ("pin_threads", c_int)]


SERVE_SYMBOLS = {
    "paella_server_start": (c_int, [ctypes.POINTER(ServerOptions), ctypes.POINTER(c_void_p)]),
    "paella_server_stop": (c_int, [c_void_p]),
    "paella_server_event_log": (c_size_t, [c_void_p, c_void_p, c_size_t]),
    "paella_server_ipc_latency": (c_int, [c_void_p, ctypes.POINTER(c_double), ctypes.POINTER(ctypes.c_uint64)]),
    "paella_ipc_latency_off": (None, []),
    "paella_client_run": (c_int, [ctypes.POINTER(LoadOptions), ctypes.POINTER(LoadResult), c_void_p]),
    "paella_direct_multistream_run": (c_int, [ctypes.POINTER(DirectOptions), ctypes.POINTER(LoadResult)]),
    "paella_workload_pregen": (c_int, [c_double, c_int, c_double, c_uint, c_uint, c_char_p, ctypes.POINTER(c_float), c_int, c_char_p, c_size_t]),
    "paella_verify_input": (c_int, [c_uint, c_uint, c_uint, c_void_p, c_size_t]),
    "paella_client_single": (c_int, [c_char_p, c_char_p, c_void_p, c_size_t, c_void_p, c_size_t, c_int, c_void_p]),
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        _abi.hip()
        path = os.path.join(_abi.LIB_DIR, "libpaella_serve.so")
        if not os.path.exists(path):
            raise RuntimeError("%s is not built: run `make -C paella_amd/csrc`" % path)
        _lib = _abi._bind(ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL), SERVE_SYMBOLS)
    return _lib


def job_path(name):
    """Absolute path of a built job definition, e.g. job_path('tvm_resnet18') or job_path('dummy_short')."""
    p = os.path.join(_abi.LIB_DIR, "libjob_%s.so" % name)
    if not os.path.exists(p):
        raise RuntimeError("%s is not built" % p)
    return p


class Server:
    """`with Server('name', 'full3', num_streams=64) as s: ...`; s.event_log() after the block."""

    def __init__(self, name, sched, num_streams=500, extra_kernels=2, unfair=1e6, sched_sleep=0, mem_marker=True, event_log=False,
                 cpu=-1, measure_block_time=False, noti_batch=0, print_ipc_latency=False, placement="pooled"):
        self.opts = ServerOptions(name.encode(), sched.encode(), num_streams, extra_kernels, unfair, sched_sleep, int(mem_marker),
                                  int(event_log), cpu, int(measure_block_time), noti_batch, int(print_ipc_latency),
                                  {"pooled": 0, "per_cu": 1}[placement])
        self.name = name
        self.handle = c_void_p()

    def __enter__(self):
        if lib().paella_server_start(ctypes.byref(self.opts), ctypes.byref(self.handle)) != 0:
            raise RuntimeError("paella_server_start failed")
        return self

    def stop(self):
        lib().paella_server_stop(self.handle)
        if self.opts.print_ipc_latency:
            lib().paella_ipc_latency_off()

    def ipc_latency(self):
        """(mean client-to-server latency of LAUNCH_JOB in us, requests it covers); needs print_ipc_latency=True."""
        mean, count = c_double(), ctypes.c_uint64()
        if lib().paella_server_ipc_latency(self.handle, ctypes.byref(mean), ctypes.byref(count)) != 0:
            raise RuntimeError("paella_server_ipc_latency failed")
        return mean.value, count.value

    def __exit__(self, *exc):
        self.stop()
        return False

    def event_log(self):
        n = lib().paella_server_event_log(self.handle, None, 0)
        buf = ctypes.create_string_buffer(n + 1)
        lib().paella_server_event_log(self.handle, buf, n + 1)
        return buf.value.decode()


def client_run(server_name, jobs, iat_us, concurrency, num_jobs, warmup_jobs=0, seed=1, dist="exp", ln_sigma=2.0, pin_threads=False,
               want_latencies=False, profile_prefix=None, trace_path=None, verify=0, expected_bytes=0):
    """jobs = [(path, proportion, max_outstanding), ...].  Returns a dict of the run's statistics.
    verify > 0: verify mode with that many seeded inputs per job type (verify_input); the dict then carries `verified_requests`
    and `mismatches`, and, when expected_bytes is given, `expected` = the outputs the idle server gave, [type][input] one after
    the other as bytes."""
    import numpy as np
    o = LoadOptions()
    o.server_name = server_name.encode()
    o.num_types = len(jobs)
    keep = []
    for i, (path, prop, mo) in enumerate(jobs):
        keep.append(path.encode())
        o.job_paths[i] = keep[-1]
        o.proportions[i] = prop
        o.max_outstanding[i] = mo
    o.iat_us, o.dist_exp, o.ln_sigma = iat_us, int(dist == "exp"), ln_sigma
    o.concurrency, o.num_jobs, o.warmup_jobs, o.seed, o.pin_threads = concurrency, num_jobs, warmup_jobs, seed, int(pin_threads)
    o.profile_prefix = profile_prefix.encode() if profile_prefix else None
    o.trace_path = trace_path.encode() if trace_path else None
    o.verify = verify
    expected = np.zeros(expected_bytes, np.uint8) if verify and expected_bytes else None
    if expected is not None:
        o.verify_expected, o.verify_expected_bytes = expected.ctypes.data, expected.nbytes
    res = LoadResult()
    lat = np.zeros(num_jobs, np.float64) if want_latencies else None
    if lib().paella_client_run(ctypes.byref(o), ctypes.byref(res), lat.ctypes.data if want_latencies else None) != 0:
        raise RuntimeError("paella_client_run failed")
    out = {"elapsed_us": res.elapsed_us, "throughput_rps": res.throughput_rps, "all": res.all.as_dict(),
           "per_type": [res.per_type[i].as_dict() for i in range(len(jobs))], "queue_full": res.queue_full_events,
           "type_full": res.type_full_events}
    if want_latencies:
        out["latencies_us"] = lat
    if verify:
        out["verified_requests"], out["mismatches"] = res.verified_requests, res.mismatches
        if expected is not None:
            out["expected"] = expected
    return out


def verify_input(seed, job_type, variant, n):
    """numpy restatement of verify mode's seeded input (csrc/serve/load_generator.h): n floats in [-1, 1)."""
    import numpy as np
    with np.errstate(over="ignore"):
        z = np.uint64((seed << 40) ^ (job_type << 32) ^ (variant << 24)) + np.arange(n, dtype=np.uint64)
        z = z + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return ((z >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / 8388608.0) - np.float32(1.0)).astype(np.float32)


def client_single(server_name, path, x, out_floats, n=1):
    """n closed-loop requests carrying input array x; returns (output array, latencies in us)."""
    import numpy as np
    x = np.ascontiguousarray(x)
    out = np.zeros(out_floats, np.float32)
    lat = np.zeros(n, np.float64)
    if lib().paella_client_single(server_name.encode(), path.encode(), x.ctypes.data, x.nbytes, out.ctypes.data, out.nbytes, n,
                                  lat.ctypes.data) != 0:
        raise RuntimeError("paella_client_single failed")
    return out, lat


def _result_dict(r, n_types):
    return {"elapsed_us": r.elapsed_us, "throughput_rps": r.throughput_rps, "all": r.all.as_dict(),
            "per_type": [r.per_type[i].as_dict() for i in range(n_types)],
            "queue_full_events": r.queue_full_events, "type_full_events": r.type_full_events}



def direct_multistream(tenants, iat_us, num_streams, num_jobs, warmup_jobs=0, seed=1, dist="exp", ln_sigma=2.0, pin_threads=False,
                       seed_weights=1):
    """Plain multi-stream serving without a server (paella_direct_multistream_run).  tenants = [(zoo model name, proportion,
    pooled instances), ...]; one stream per request in flight."""
    o = DirectOptions()
    o.num_types = len(tenants)
    keep = []
    for i, (model, prop, mo) in enumerate(tenants):
        keep.append(model.encode())
        o.models[i] = keep[-1]
        o.proportions[i] = prop
        o.max_outstanding[i] = mo
    o.seed_weights, o.num_streams, o.iat_us, o.dist_exp, o.ln_sigma = seed_weights, num_streams, iat_us, int(dist == "exp"), ln_sigma
    o.num_jobs, o.warmup_jobs, o.seed, o.pin_threads = num_jobs, warmup_jobs, seed, int(pin_threads)
    r = LoadResult()
    if lib().paella_direct_multistream_run(ctypes.byref(o), ctypes.byref(r)) != 0:
        raise RuntimeError("paella_direct_multistream_run failed")
    return _result_dict(r, len(tenants))


def workload_pregen(prefix, proportions, iat_us, num_jobs, seed=1, dist="ln", ln_sigma=1.5):
    """Writes an arrival trace (paella_workload_pregen); returns the combined file's path."""
    props = (c_float * len(proportions))(*proportions)
    buf = ctypes.create_string_buffer(4096)
    if lib().paella_workload_pregen(iat_us, int(dist == "exp"), ln_sigma, num_jobs, seed, str(prefix).encode(), props, len(proportions), buf, 4096) != 0:
        raise RuntimeError("paella_workload_pregen failed")
    return buf.value.decode()
