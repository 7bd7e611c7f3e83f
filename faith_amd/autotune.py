"""Kernel-variant autotuner: heuristics propose, a cost model ranks, the GPU decides.

Counterpart of the reference's autotuner (autotuner/autotuner.py:99-147: rounds of sampling, the
first at random and the later ones ranked by a learned cost model; expert_knowledge_metafile.py:
16-80, :96-190: a hardware "metafile" and validity heuristics such as "the block tile fits in
shared memory" and "the warp tile fits in registers"; cost_model.py: a regressor on
[implementation parameters + metafile]).  The reference rewrites matmul_config.h and recompiles
for every sample; here the variants are template instantiations that are already in
libfaith_amd.so and are selected per call through faith_tune_set, so a sample costs a few launches.

What can be tuned (see the FAITH_TUNE_* knobs in include/faith_amd.h):

    linear       macro-tile of the sign-split GEMM: 64x64, 128x128, 128x64, 64x128, or 32x32 with the
                 reduction split over the workgroup's wavefronts
    dot_qk/dot_v 128x64 persistent tiles, or one 32x32 block per wavefront with 1..16 perturbation
                 coordinates per wavefront
    act          tile shape of the relaxation kernels (relu, tanh, exp, ...)
    concretize   tile shape of the concretize kernel

Results are kept in a TuningTable keyed by (operator, shape); `use(table)` makes the wrappers in
faith_amd.ops apply an entry around the matching launch.  Results never depend on the variant, only
speed does.

Beyond the variants the library ships, `autotune_generated` runs the reference's loop as it is: a variant of the
GEMM's MFMA kernel -- tile shape, register budget, wavefront priority, i.e. what matmul_config.h holds there -- is
GENERATED as macros, COMPILED with hipcc into a small library of its own (csrc/variants/gemm_variant.hip, a few
seconds), loaded, checked against the shipped kernel bit for bit and measured; the table then names the compiled
library and faith_amd.ops.linear sends the coefficient rows of that shape through it.
"""
from __future__ import annotations

import contextlib
import ctypes
import hashlib
import json
import os
import random
import shutil
import subprocess
from dataclasses import dataclass, field

import numpy as np

# knob numbers of include/faith_amd.h
TUNE_ACT_VARIANT, TUNE_GEMM_VARIANT, TUNE_DOT_VARIANT, TUNE_DOT_COORDS = 0, 1, 2, 3

# Hardware description the heuristics and the cost model see (the reference's a100_metafile).
mi355x_metafile = {
    "COMPUTE_UNITS": 256,
    "MAX_LDS_KB": 160,              # per compute unit
    "MAX_NUM_REGISTER_PER_LANE": 512,   # vector + accumulator registers of one wavefront
    "MAX_WAVES_PER_SIMD": 8,
    "SIMDS_PER_CU": 4,
    "XCDS": 8,
}


def metafile_of_device(index=0):
    """The metafile with the compute-unit count of the GPU that is present."""
    import torch
    m = dict(mi355x_metafile)
    m["COMPUTE_UNITS"] = torch.cuda.get_device_properties(index).multi_processor_count
    return m


@dataclass(frozen=True)
class Candidate:
    """One implementation choice: knob settings plus the quantities the heuristics reason about."""
    knobs: tuple                    # ((knob, value), ...)
    params: tuple                   # ((name, number), ...): tile sizes, LDS bytes, registers, ...

    def knob_dict(self):
        return dict(self.knobs)

    def param(self, name, default=0.0):
        return dict(self.params).get(name, default)


def _cand(knobs, **params):
    return Candidate(tuple(sorted(knobs.items())), tuple(sorted(params.items())))


class Heuristics:
    """Proposes candidates for an (operator, shape) and rejects the ones that cannot be good
    (expert_knowledge_metafile.py:36-190 plays this role for the CUTLASS tile parameters)."""

    OPERATORS = ("linear", "dot_qk", "dot_v", "act", "concretize")

    def __init__(self, metafile=None):
        self.metafile = dict(mi355x_metafile if metafile is None else metafile)

    # ---- checks shared by the operators
    def check_lds(self, lds_bytes):
        return lds_bytes <= self.metafile["MAX_LDS_KB"] * 1024

    def check_registers(self, registers_per_lane):
        return registers_per_lane <= self.metafile["MAX_NUM_REGISTER_PER_LANE"]

    def resident_workgroups(self, lds_bytes, registers_per_lane, waves_per_group=4):
        """Workgroups one compute unit can hold at a time."""
        by_lds = (self.metafile["MAX_LDS_KB"] * 1024) // max(lds_bytes, 1)
        waves = min(self.metafile["MAX_WAVES_PER_SIMD"],
                    self.metafile["MAX_NUM_REGISTER_PER_LANE"] // max(registers_per_lane, 1))
        by_regs = waves * self.metafile["SIMDS_PER_CU"] // waves_per_group
        return max(0, min(by_lds, by_regs))

    # ---- proposals
    def propose(self, op, shape):
        """All candidates for the operator, valid or not."""
        if op == "linear":
            rows, k, n = shape
            out = []
            for variant, (tm, tn) in {1: (64, 64), 2: (128, 128), 3: (128, 64), 4: (64, 128)}.items():
                lds = 2 * 2 * 16 * (tm + tn) * 4            # two stages; A_l, A_u [tm x 16] and W+, W- [tn x 16] floats
                acc = 2 * (tm // 2) * (tn // 2) // 64 * 1   # accumulator registers per lane for C_l and C_u
                tiles = -(-rows // tm) * -(-n // tn)
                out.append(_cand({TUNE_GEMM_VARIANT: variant}, tile_m=tm, tile_n=tn, lds_bytes=lds,
                                 registers=acc + 40 + 12 * (tm + tn) // 64, workgroups=tiles,
                                 padding=(-(-rows // tm) * tm * -(-n // tn) * tn) / float(rows * n) - 1.0,
                                 steps=-(-k // 16), mfma_per_step=(tm // 64) * (tn // 64) * 32))
            # 32 x 32 block per workgroup, the reduction split over its four wavefronts (tiny problems)
            out.append(_cand({TUNE_GEMM_VARIANT: 5}, tile_m=32, tile_n=32, lds_bytes=32768, registers=140,
                             workgroups=-(-rows // 32) * -(-n // 32),
                             padding=(-(-rows // 32) * 32 * -(-n // 32) * 32) / float(rows * n) - 1.0,
                             steps=-(-k // 32), mfma_per_step=16))
            return out
        if op in ("dot_qk", "dot_v"):
            batch, lx, ly, d_in, d = shape
            out = [_cand({TUNE_DOT_VARIANT: 1}, tile_m=128, tile_n=64, lds_bytes=2 * (4 * 128 + 6 * 64) * 8 * 4,
                         registers=232, workgroups=batch * d_in * -(-lx // 128) * -(-ly // 64),
                         padding=(-(-lx // 128) * 128 * -(-ly // 64) * 64) / float(lx * ly) - 1.0,
                         steps=-(-d // 8), mfma_per_step=64, coords=0)]
            blocks = batch * -(-lx // 32) * -(-ly // 32)
            for coords in (1, 2, 3, 4, 6, 8, 12, 16):
                out.append(_cand({TUNE_DOT_VARIANT: 2, TUNE_DOT_COORDS: coords}, tile_m=32, tile_n=32,
                                 lds_bytes=6 * 32 * d * 4, registers=166,
                                 workgroups=blocks * -(-d_in // (4 * coords)),
                                 padding=(-(-lx // 32) * 32 * -(-ly // 32) * 32) / float(lx * ly) - 1.0,
                                 steps=-(-d // 8) * coords, mfma_per_step=32, coords=coords))
            return out
        if op == "act":
            rows, d_in, h = shape
            table = {0: (32, 32, 256), 9: (32, 256, 256), 1: (32, 256, 256), 2: (64, 256, 512), 3: (64, 256, 1024),
                     4: (32, 256, 512), 5: (64, 256, 256), 6: (32, 1024, 1024)}   # neurons per tile, rows per pass, threads
            out = []
            for variant, (neurons, chunk, threads) in table.items():
                held = min(d_in, chunk) * neurons * 2 // threads       # values a thread keeps between its two passes
                out.append(_cand({TUNE_ACT_VARIANT: variant}, tile_n=neurons, chunk=chunk, threads=threads,
                                 registers=held + 40, lds_bytes=8 * neurons * (threads // 64),
                                 workgroups=rows * -(-h // neurons), resident=1.0 if variant == 0 else 0.0))
            return out
        if op == "concretize":
            rows, d_in, h = shape
            return [_cand({TUNE_ACT_VARIANT: v}, tile_n=n, threads=t, registers=48, lds_bytes=8 * n * (t // 64),
                          workgroups=rows * -(-h // n))
                    for v, (n, t) in {0: (64, 1024), 11: (64, 256), 13: (32, 256)}.items()]
        raise ValueError(f"unknown operator {op!r}; one of {self.OPERATORS}")

    def is_valid(self, op, shape, cand):
        """Fits the machine and is not mostly padding."""
        if not self.check_lds(cand.param("lds_bytes")) or not self.check_registers(cand.param("registers")):
            return False
        if op == "linear":
            # a tile more than twice the problem in either direction is padding only
            rows, k, n = shape
            if cand.knob_dict().get(TUNE_GEMM_VARIANT) == 5:
                return k % 32 == 0            # each wavefront takes a quarter of K in steps of 8
            return cand.param("tile_m") < 2 * max(rows, 64) and cand.param("tile_n") < 2 * max(n, 64)
        if op in ("dot_qk", "dot_v"):
            _, lx, ly, _, d = shape
            if cand.knob_dict().get(TUNE_DOT_VARIANT) == 2:
                # the per-wavefront kernel keeps the six sign-split operands of the whole reduction in LDS
                return d % 8 == 0 and d <= 80 and cand.param("padding") < 1.0
            return True
        if op == "act":
            _, d_in, h = shape
            if cand.knob_dict().get(TUNE_ACT_VARIANT) == 0:
                return True                                  # the built-in choice is always available
            return h % 4 == 0
        return True

    def candidates(self, op, shape):
        return [c for c in self.propose(op, shape) if self.is_valid(op, shape, c)]

    # ---- features for the cost model: implementation parameters, shape, metafile
    FEATURES = ("tile_m", "tile_n", "lds_bytes", "registers", "workgroups", "padding", "steps", "mfma_per_step",
                "coords", "chunk", "threads", "resident")

    def features(self, op, shape, cand):
        cus = self.metafile["COMPUTE_UNITS"]
        resident = self.resident_workgroups(cand.param("lds_bytes"), cand.param("registers"))
        rounds = cand.param("workgroups") / float(max(1, resident * cus))
        own = [float(cand.param(name)) for name in self.FEATURES]
        derived = [rounds, float(np.ceil(rounds)), float(resident)]
        return np.array(own + derived + [float(s) for s in shape] + [float(v) for v in self.metafile.values()])


class CostModel:
    """Ridge regression of log-latency on standardised features (the reference trains an XGBoost
    regressor, cost_model.py:15-21; with a handful of samples per shape a linear model ranks as well
    and needs nothing beyond numpy)."""

    def __init__(self, ridge=1e-2):
        self.ridge = ridge
        self.mean = self.scale = self.weights = None

    def fit(self, features, latencies):
        x = np.asarray(features, dtype=np.float64)
        y = np.log(np.asarray(latencies, dtype=np.float64))
        self.mean = x.mean(axis=0)
        self.scale = x.std(axis=0)
        self.scale[self.scale == 0] = 1.0
        z = np.hstack([(x - self.mean) / self.scale, np.ones((x.shape[0], 1))])
        reg = self.ridge * np.eye(z.shape[1])
        reg[-1, -1] = 0.0
        self.weights = np.linalg.solve(z.T @ z + reg, z.T @ y)
        return self

    def predict(self, features):
        x = np.atleast_2d(np.asarray(features, dtype=np.float64))
        z = np.hstack([(x - self.mean) / self.scale, np.ones((x.shape[0], 1))])
        return np.exp(z @ self.weights)


def measure_on_gpu(run, repeats=15, inner=4, warm_seconds=0.03):
    """Latency of run() in microseconds: `inner` launches back to back between one pair of events on
    the current stream, median over `repeats` such groups, after warming up by time (clocks take
    milliseconds to rise after idle)."""
    import time
    import torch
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < warm_seconds:
        run()
    torch.cuda.synchronize()
    times = []
    for _ in range(repeats):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(inner):
            run()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b) * 1e3 / inner)
    return float(np.median(times))


def _set_knobs(knobs, setter=None):
    if setter is None:
        from . import _lib
        setter = lambda k, v: _lib.call("faith_tune_set", int(k), int(v))
    for k, v in knobs.items():
        setter(k, v)


@contextlib.contextmanager
def applied(knobs, setter=None):
    """Sets the knobs for the duration of the block and restores the built-in choices afterwards."""
    _set_knobs(knobs, setter)
    try:
        yield
    finally:
        _set_knobs({k: 0 for k in knobs}, setter)


@dataclass
class TuningResult:
    op: str
    shape: tuple
    best: Candidate
    best_us: float
    measured: list = field(default_factory=list)       # [(Candidate, microseconds)], in the order measured
    skipped: int = 0


def autotune(op, shape, run, heuristics=None, rounds=3, samples=3, measure=None, setter=None, seed=0):
    """Finds the fastest valid candidate for run() -- a callable that launches the operator once.

    The first tuning round measures `samples` candidates drawn at random; every later one fits the cost model to
    what has been measured and measures the `samples` unmeasured candidates it predicts to be fastest
    (autotuner.py:99-147).  The built-in choice (all knobs 0) is always among the measured ones, so the
    result is never slower than not tuning.  measure(run) -> microseconds defaults to GPU events."""
    heuristics = heuristics or Heuristics()
    measure = measure or measure_on_gpu
    rng = random.Random(seed)
    pool = heuristics.candidates(op, shape)
    if not pool:
        raise ValueError(f"no valid candidate for {op} {shape}")
    result = TuningResult(op, tuple(shape), None, float("inf"))
    seen = set()

    def take(cand):
        seen.add(cand)
        try:
            with applied(cand.knob_dict(), setter):
                us = measure(run)
        except Exception:                                   # a variant that cannot run this shape
            result.skipped += 1
            return
        result.measured.append((cand, us))
        if us < result.best_us:
            result.best, result.best_us = cand, us

    try:
        measure(run)        # discarded: the first measurement after idle runs at lower clocks
    except Exception:
        pass
    builtin = Candidate((), (("builtin", 1.0),))
    take(builtin)
    for r in range(rounds):
        rest = [c for c in pool if c not in seen]
        if not rest:
            break
        fitted = [(c, us) for c, us in result.measured if c is not builtin]
        if r == 0 or len(fitted) < 2:
            chosen = rng.sample(rest, min(samples, len(rest)))
        else:
            model = CostModel().fit([heuristics.features(op, shape, c) for c, _ in fitted], [us for _, us in fitted])
            ranked = sorted(rest, key=lambda c: float(model.predict(heuristics.features(op, shape, c))[0]))
            chosen = ranked[:samples]
        for cand in chosen:
            take(cand)
    return result


# ------------------------------------------------------------------------------------------
# Generated variants: generate -> compile -> load -> measure (autotuner.py:99-147 with
# utils.py's rewrite-and-rebuild step; here the rebuilt unit is one translation unit, not the extension)
# ------------------------------------------------------------------------------------------
_HERE = os.path.dirname(os.path.abspath(__file__))
VARIANT_SOURCE = os.path.join(_HERE, "csrc", "variants", "gemm_variant.hip")


@dataclass(frozen=True)
class GemmVariantSpec:
    """What one generated GEMM kernel is compiled with: 32 x 32 MFMA blocks per wavefront along M and N (the
    macro-tile is 64 mbm x 64 mbn), wavefronts per SIMD the register budget is set for, raised wavefront priority
    during a run of MFMAs."""
    mbm: int
    mbn: int
    waves: int
    setprio: int

    def macros(self):
        return {"FAITH_V_MBM": self.mbm, "FAITH_V_MBN": self.mbn, "FAITH_V_WAVES": self.waves,
                "FAITH_GEMM_SETPRIO": self.setprio}

    def lds_bytes(self):
        return 2 * (4 * 64 * self.mbm * 8 + 4 * 64 * self.mbn * 8) * 4

    def registers(self):
        return 2 * 16 * self.mbm * self.mbn + 8 * (self.mbm + self.mbn) + 40     # accumulators, fragments, the rest

    def name(self):
        return f"gemm_{64 * self.mbm}x{64 * self.mbn}_w{self.waves}_p{self.setprio}"


def gemm_variant_space(metafile=None):
    """Every variant the tile code can express and the part can hold: the accumulators of both operands fit a
    wavefront's share of the registers at the asked-for occupancy, the two LDS stages fit a workgroup."""
    meta = dict(mi355x_metafile, **(metafile or {}))
    out = []
    for mbm in (1, 2, 3, 4):
        for mbn in (1, 2, 3, 4):
            if mbm * mbn > 4:
                continue
            for waves in (1, 2, 3, 4):
                for setprio in (0, 1):
                    v = GemmVariantSpec(mbm, mbn, waves, setprio)
                    if v.lds_bytes() > meta["MAX_LDS_KB"] * 1024:
                        continue
                    if v.registers() > meta["MAX_NUM_REGISTER_PER_LANE"] // waves:
                        continue
                    out.append(v)
    return out


def compile_gemm_variant(spec, out_dir, hipcc="hipcc", arch="gfx950"):
    """Compiles the variant into out_dir and returns the library's path (an existing build of the same source and
    macros is reused).  Needs hipcc; a GPU is not needed to build."""
    if shutil.which(hipcc) is None:
        raise RuntimeError(f"{hipcc} not found: generated variants are compiled on the machine that tunes")
    os.makedirs(out_dir, exist_ok=True)
    src = open(VARIANT_SOURCE, "rb").read() + open(os.path.join(_HERE, "csrc", "gemm_tile.h"), "rb").read()
    tag = hashlib.sha256(src + json.dumps(spec.macros(), sort_keys=True).encode()).hexdigest()[:12]
    path = os.path.join(out_dir, f"libfaith_{spec.name()}_{tag}.so")
    if os.path.exists(path):
        return path
    from .build import COMMON
    cmd = [hipcc, *COMMON, *[f"-D{k}={v}" for k, v in spec.macros().items()], "-shared", VARIANT_SOURCE,
           os.path.join(_HERE, "csrc", "common.hip"), "-o", path + ".tmp"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {spec.name()}:\n{r.stderr[-2000:]}")
    os.replace(path + ".tmp", path)
    return path


class GeneratedGemm:
    """A compiled variant, loaded.  coefficients(...) multiplies the coefficient rows of a layer; the constant
    rows stay with the library's exact-accumulation kernel (faith_matmul_rows_verification with no coefficient
    rows)."""

    def __init__(self, path):
        self.path = path
        self.lib = ctypes.CDLL(path)
        P, I = ctypes.c_void_p, ctypes.c_int
        self.lib.faith_variant_matmul_coefficients.argtypes = [P] * 5 + [ctypes.c_longlong, I, I, P]
        self.lib.faith_variant_matmul_coefficients.restype = I
        self.lib.faith_last_error.restype = ctypes.c_char_p
        self.lib.faith_variant_lds_bytes.restype = I

    def coefficients(self, lw, uw, weight, olw, ouw, stream):
        rows = lw.numel() // lw.shape[-1]
        rc = self.lib.faith_variant_matmul_coefficients(lw.data_ptr(), uw.data_ptr(), weight.data_ptr(), olw.data_ptr(),
                                                        ouw.data_ptr(), rows, lw.shape[-1], weight.shape[0], stream)
        if rc != 0:
            from ._lib import FaithError
            raise FaithError("faith_variant_matmul_coefficients", rc, self.lib.faith_last_error().decode())


_LOADED = {}


def load_generated(path):
    g = _LOADED.get(path)
    if g is None:
        g = _LOADED[path] = GeneratedGemm(path)
    return g


def autotune_generated(shape, lw, uw, weight, out_dir, specs=None, rounds=3, samples=4, measure=None, seed=0,
                       compile_variant=compile_gemm_variant):
    """The generate-and-recompile loop for the coefficient rows of `linear` at shape = (rows, K, N):
    lw, uw [..., K] and weight [N, K] are the operands to measure on (GPU tensors).

    Round 0 compiles and measures `samples` specs drawn at random, later rounds the `samples` unmeasured specs the
    cost model (fitted on what has been measured) ranks fastest.  The shipped kernel is measured first and a
    generated variant is only kept if it is faster -- measured as ops.linear would run it, the launch for the
    constant rows included -- AND reproduces the shipped kernel's coefficient rows bit for bit (the order of
    summation does not depend on the tile).  Returns (TuningResult, path of the best library or
    None if the shipped kernel stays)."""
    import torch
    from . import _lib, ops
    measure = measure or measure_on_gpu
    rng = random.Random(seed)
    pool = list(specs) if specs is not None else gemm_variant_space()
    rows, K, N = (int(v) for v in shape)
    x_lw, x_uw = lw.reshape(1, 1, rows, K), uw.reshape(1, 1, rows, K)
    zeros_b = torch.zeros(1, 1, K, device=lw.device)
    ref = ops.linear(x_lw, zeros_b, x_uw, zeros_b, weight)
    olw, ouw = torch.empty_like(ref[0]), torch.empty_like(ref[2])
    stream = torch.cuda.current_stream(lw.device).cuda_stream
    result = TuningResult("linear", (rows, K, N), None, float("inf"))
    builtin = Candidate((), (("builtin", 1.0),))
    out4 = (ref[0], ref[1], ref[2], ref[3])
    shipped = lambda: ops.linear(x_lw, zeros_b, x_uw, zeros_b, weight, out=out4)
    measure(shipped)                                    # discarded: clocks
    result.best, result.best_us = builtin, measure(shipped)
    result.measured.append((builtin, result.best_us))
    best_path = None
    seen = set()

    def feats(v):
        tiles = -(-rows // (64 * v.mbm)) * -(-N // (64 * v.mbn))
        resident = max(1, min(v.waves, (160 * 1024) // v.lds_bytes())) * mi355x_metafile["COMPUTE_UNITS"]
        return [1.0, v.mbm, v.mbn, v.mbm * v.mbn, v.waves, v.setprio, np.log(tiles), np.ceil(tiles / resident)]

    def take(v):
        nonlocal best_path
        seen.add(v)
        try:
            g = load_generated(compile_variant(v, out_dir))

            def run():      # what ops.linear does with a generated entry: the variant, then the constant rows
                g.coefficients(x_lw, x_uw, weight, olw, ouw, stream)
                _lib.call("faith_matmul_rows_verification", zeros_b.data_ptr(), zeros_b.data_ptr(), None, None,
                          weight.data_ptr(), None, ref[1].data_ptr(), ref[3].data_ptr(), None, None, 0, 1, K, N, stream)
            run()
            torch.cuda.synchronize(lw.device)
            if not (torch.equal(olw, ref[0]) and torch.equal(ouw, ref[2])):
                raise RuntimeError("results differ from the shipped kernel's")
            us = measure(run)
        except Exception:
            result.skipped += 1
            return
        cand = _cand({}, **{k.lower(): float(val) for k, val in v.macros().items()})
        result.measured.append((cand, us))
        spec_of[cand] = v
        if us < result.best_us:
            result.best, result.best_us, best_path = cand, us, g.path

    spec_of = {}
    for r in range(rounds):
        rest = [v for v in pool if v not in seen]
        if not rest:
            break
        fitted = [(spec_of[c], us) for c, us in result.measured if c in spec_of]
        if r == 0 or len(fitted) < 3:
            chosen = rng.sample(rest, min(samples, len(rest)))
        else:
            model = CostModel().fit([feats(v) for v, _ in fitted], [us for _, us in fitted])
            chosen = sorted(rest, key=lambda v: float(model.predict([feats(v)])[0]))[:samples]
        for v in chosen:
            take(v)
    return result, best_path


class TuningTable:
    """(operator, shape) -> knob settings; JSON on disk."""

    def __init__(self):
        self.entries = {}

    @staticmethod
    def key(op, shape):
        return f"{op}:" + "x".join(str(int(s)) for s in shape)

    def record(self, result):
        self.entries[self.key(result.op, result.shape)] = {
            "knobs": {str(k): int(v) for k, v in result.best.knob_dict().items()},
            "microseconds": round(result.best_us, 2),
            "measured": len(result.measured)}

    def record_generated(self, result, path):
        """The outcome of autotune_generated: the compiled library for this shape, or the shipped kernel."""
        self.entries[self.key(result.op, result.shape)] = {
            "knobs": {}, "microseconds": round(result.best_us, 2), "measured": len(result.measured),
            **({"generated": path} if path else {})}

    def lookup(self, op, shape):
        e = self.entries.get(self.key(op, shape))
        return None if e is None else {int(k): int(v) for k, v in e["knobs"].items()}

    def generated(self, op, shape):
        """Path of the compiled variant recorded for (op, shape), or None."""
        e = self.entries.get(self.key(op, shape))
        return None if e is None else e.get("generated")

    def save(self, path):
        with open(path, "w") as f:
            json.dump(self.entries, f, indent=1, sort_keys=True)

    @classmethod
    def load(cls, path):
        t = cls()
        with open(path) as f:
            t.entries = json.load(f)
        return t


_ACTIVE = None


def use(table):
    """Makes faith_amd.ops apply `table` (None: stop)."""
    global _ACTIVE
    _ACTIVE = table
