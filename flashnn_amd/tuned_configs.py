"""Shape-keyed tuned configurations with an on-disk JSON file - the role that
compile_and_cache_kernels and configs/triton_autotune_best_configs.json play in the reference
(flashnn/triton_kernels/triton_utils.py:14-24, 38-80, 84-151).

A kernel launch is named by a method name ("gemm_a8w8_M_N_K", the reference's own,
triton_kernels/gemm_a8w8.py:199; the weight-only GEMMs of up to 64 rows, which the reference tunes in-process
by M, N, K - gemm_a16w8.py:322-336 - are named after its kernels: "gemm_a16w8_per_channel_M_N_K",
"gemm_a16w4_sub_channel_g128_M_N_K").  The first time a method name is met while tuning is switched on
(set_autotune_triton_kernels(True), as in the reference) the candidates are timed on the caller's
operands and the best one is recorded, in memory and in the JSON file; afterwards, and in later
processes, the recorded configuration is used without timing anything.  With tuning switched off
recorded configurations are still honoured; shapes without one take the library's static choice.

File format (the reference's, triton_utils.py:38-57): {method_name: [kwargs, launch_options]} with
kwargs = {"BLOCK_M": .., "BLOCK_N": ..} ((0, 0) = the library's own choice, its own split of K included), an
optional "SPLIT_K": n (K cut into n parts per tile, met through the launcher's workspace; the name the
reference's weight-only kernels give the notion, gemm_a16w8.py:17-80; absent = 1) and launch_options =
{"num_warps": 4} (absent = the tile's default; every tile runs four waves), the reference's own option names (gemm_a8w8.py:17-50).
The file lives at $FLASHNN_AMD_TUNED_CONFIGS or flashnn_amd/configs/hip_autotune_best_configs.json.
FORECE_RE_TUNE_TRITON_KERNELS (the reference's spelling, triton_utils.py:22-24) lists method-name
prefixes, separated by ';', that are tuned again even if recorded.
"""
import json
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
JSON_FILENAME = "hip_autotune_best_configs.json"

# candidate (rows, columns, waves, parts of K) of the A8W8 MFMA kernel; (0, 0, 0, 0) = static choice (which may
# be a few-row kernel, or a split of its own); waves = 0 is the tile's default (four).  Splits a shape does not
# admit (parts shorter than four slabs, M or N too small) are refused by the library and skipped by tune().
A8W8_CANDIDATES = [(0, 0, 0, 0), (256, 256, 0, 1), (256, 192, 0, 1), (256, 128, 0, 1), (128, 128, 0, 1), (64, 128, 0, 1),
                   (128, 128, 0, 2), (128, 128, 0, 3), (128, 128, 0, 4), (128, 128, 0, 6), (128, 128, 0, 8)]


def weight_only_candidates(channels_per_weight_row):
    """Candidate (rows per pass, channels per workgroup, 0, 1) of the few-row weight-only kernel, the BLOCK_M and
    BLOCK_N of the reference's lists (gemm_a16w8.py:15-80, gemm_a16w4.py:15-80); (0, 0, 0, 0) = the library's
    choice, which comes first because every shape admits it.  A workgroup takes 16, 32 or 64 weight rows (one or
    two channels each) and at most as many activation rows per pass; pairs a shape does not divide into are
    refused by the library and skipped by tune()."""
    c = channels_per_weight_row
    return [(0, 0, 0, 0)] + [(16 * mb, 16 * rt * c, 0, 1) for rt in (4, 2, 1) for mb in (4, 2, 1) if mb <= rt]


def as_config(tile):
    """(rows, columns[, waves[, parts]]) -> the full 4-tuple; a named tile without parts is unsplit."""
    t = tuple(int(v) for v in tile)
    t = t + (0,) * (3 - len(t)) if len(t) < 3 else t
    if len(t) == 3:
        t = t + ((1,) if t[0] else (0,))
    return t


def json_file_path():
    return os.environ.get("FLASHNN_AMD_TUNED_CONFIGS") or os.path.join(_HERE, "configs", JSON_FILENAME)


def _force_list():
    return [k for k in os.getenv("FORECE_RE_TUNE_TRITON_KERNELS", "None").split(";") if k]


def force_re_tune(method_name):
    return any(method_name.startswith(kernel) for kernel in _force_list())


def serialize_best_config(tile):
    bm, bn, waves, parts = as_config(tile)
    kwargs = {"BLOCK_M": bm, "BLOCK_N": bn}
    if parts > 1:
        kwargs["SPLIT_K"] = parts
    return [kwargs, {"num_warps": waves} if waves else {}]


def deserialize_best_config(entry):
    kwargs, options = entry[0], entry[1] if len(entry) > 1 else {}
    bm = int(kwargs["BLOCK_M"])
    return bm, int(kwargs["BLOCK_N"]), int(options.get("num_warps", 0)), int(kwargs.get("SPLIT_K", 1 if bm else 0))


class TunedConfigs:
    """In-memory view of the JSON file (read once per path; written through on every new record).

    shape_tile() is what a launcher calls on every GEMM: it answers from a dictionary keyed by the shape and
    touches neither the environment nor the file once a shape has been resolved.  The environment (file
    path, forced re-tune list) is therefore read when a shape is first met; after changing it inside a
    running process call reset()."""

    def __init__(self):
        self._path = None
        self._data = {}
        self._tuned_now = set()      # method names tuned by this process (a forced re-tune runs once)
        self._by_shape = {}          # (prefix, M, N, K) -> tile or None, resolved once

    def reset(self):
        """Forget everything read so far: the next lookup reads the environment and the file again."""
        self.__init__()

    def shape_tile(self, prefix, M, N, K):
        """The recorded tile for "<prefix>_M_N_K", or None; resolved once per shape."""
        key = (prefix, M, N, K)
        try:
            return self._by_shape[key]
        except KeyError:
            tile = self._by_shape[key] = self.lookup(f"{prefix}_{M}_{N}_{K}")
            return tile

    def _load(self):
        path = json_file_path()
        if path != self._path:
            self._path = path
            self._data = {}
            self._tuned_now = set()
            if os.path.exists(path):
                with open(path, "r", encoding="utf-8") as f:
                    self._data = json.load(f)
        return self._data

    def lookup(self, method_name):
        """The recorded tile of `method_name`, or None (also when a re-tune is forced and still due)."""
        data = self._load()
        if method_name not in data:
            return None
        if force_re_tune(method_name) and method_name not in self._tuned_now:
            return None
        return deserialize_best_config(data[method_name])

    def record(self, method_name, tile):
        data = self._load()
        data[method_name] = serialize_best_config(tile)
        self._tuned_now.add(method_name)
        self._by_shape.clear()
        os.makedirs(os.path.dirname(self._path), exist_ok=True)
        tmp = self._path + ".tmp"
        with open(tmp, "w", encoding="utf-8") as f:
            json.dump(data, f, indent=4)
        os.replace(tmp, self._path)


CACHE = TunedConfigs()


def tune(method_name, candidates, run, reps=5):
    """Times run(candidate) for every candidate with GPU events (one warm-up call, then the median of
    `reps` calls each), records and returns the fastest.  A candidate the library refuses for this shape
    (run raises) is skipped; the first candidate must be one that every shape admits."""
    import torch
    best, best_ms = candidates[0], float("inf")
    for n, cand in enumerate(candidates):
        try:
            run(cand)
        except Exception:
            if n == 0:
                raise
            continue
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            run(cand)
            e.record()
            e.synchronize()
            times.append(s.elapsed_time(e))
        ms = sorted(times)[len(times) // 2]
        if ms < best_ms:
            best, best_ms = cand, ms
    CACHE.record(method_name, best)
    return best
