"""Synthetic inputs for the five workloads the path is measured and tested on.

Each generator is a pure function of (seed, shape): numpy's counter-based
Philox stream keyed by the seed, so the host oracle, the tests and the device
benchmark regenerate identical bits without shipping tensors.  All arithmetic
that shapes the data is done in float32 on the host, so the kernel and the
oracle see the same bit patterns.
"""
import numpy as np

SEEDS = {"C1": 1001, "C2": 1002, "C3": 1003, "C4": 1004, "C5": 1005}


def _rng(seed):
    return np.random.Generator(np.random.Philox(key=int(seed)))


def classifier_logits(rows=1, cols=1000, seed=SEEDS["C1"]):
    """C1 / C2: classifier-head logits ~ N(0, 3^2), float32 [rows, cols]."""
    g = _rng(seed)
    return (g.standard_normal((rows, cols), dtype=np.float32) * np.float32(3.0)).astype(np.float32)


def llm_logits(rows=64, cols=128256, seed=SEEDS["C3"], temperature=0.8):
    """C3: vocabulary logits ~ N(0,1) with 1-3 spikes per row of +6..+10,
    then scaled by 1/temperature in float32."""
    g = _rng(seed)
    x = g.standard_normal((rows, cols), dtype=np.float32)
    for r in range(rows):
        ns = int(g.integers(1, 4))
        pos = g.choice(cols, size=ns, replace=False)
        x[r, pos] += g.uniform(6.0, 10.0, size=ns).astype(np.float32)
    x *= np.float32(1.0 / temperature)
    return x


def grid_values(rows=8, cols=262144, seed=SEEDS["C4"]):
    """C4: values on the 513-point grid {-4, -4+1/64, ..., 4}: many exact ties."""
    g = _rng(seed)
    q = g.integers(0, 513, size=(rows, cols), dtype=np.int32) - 256
    return (q.astype(np.float32) / np.float32(64.0)).astype(np.float32)


def detection_scores(batch=16, classes=80, anchors=8400, seed=SEEDS["C5"]):
    """C5: detection-head class scores ~ N(-4, 2^2), float32 [batch, classes, anchors]."""
    g = _rng(seed)
    x = g.standard_normal((batch, classes, anchors), dtype=np.float32)
    return (x * np.float32(2.0) - np.float32(4.0)).astype(np.float32)


AWKWARD_KINDS = ["normal", "ascending", "descending", "constant", "two_values", "levels", "masked_90", "three_allowed", "nan_row",
                 "inf_row", "flat_with_peaks", "runs", "bf16_valued", "times_1e4"]


def awkward_rows(kind, rows, cols, seed=7):
    """Rows that are hard on a selection kernel, for the data sweep of the operator
    bench and for tests: float32 [rows, cols] of N(0, 1.25^2) values, reshaped into
    sorted rows, rows of one or two values, a dozen levels, rows of mostly -inf, rows
    with a NaN or +inf, one value with a few peaks, rows sorted in runs of 4096,
    bfloat16-valued and very spread-out (x 1e4) logits."""
    g = _rng(seed)
    x = (g.standard_normal((rows, cols), dtype=np.float32) * np.float32(1.25)).astype(np.float32)
    if kind == "normal":
        return x
    if kind == "ascending":
        return np.sort(x, axis=1)
    if kind == "descending":
        return np.ascontiguousarray(-np.sort(-x, axis=1))
    if kind == "constant":
        return np.full((rows, cols), 0.75, np.float32)
    if kind == "two_values":
        return np.where(x > 0, np.float32(1.0), np.float32(-1.0)).astype(np.float32)
    if kind == "levels":
        return (np.round(x * 2) / 2).astype(np.float32)
    if kind == "masked_90":
        x[g.random((rows, cols)) < 0.9] = -np.inf
        return x
    if kind == "three_allowed":
        x[:] = -np.inf
        x[:, :3] = 0.5
        return x
    if kind == "nan_row":
        x[0, cols // 2] = np.nan
        return x
    if kind == "inf_row":
        x[0, cols // 3] = np.inf
        return x
    if kind == "flat_with_peaks":
        x[:] = np.float32(-0.3)
        m = min(cols // 2, 1100)
        for r in range(rows):
            x[r, g.choice(cols, m, replace=False)] = g.standard_normal(m, dtype=np.float32) + np.float32(3.0)
        return x
    if kind == "runs":
        return np.concatenate([np.sort(x[:, i:i + 4096], axis=1) for i in range(0, cols, 4096)], axis=1)
    if kind == "bf16_valued":
        return np.ascontiguousarray((x.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32))
    if kind == "times_1e4":
        return (x * np.float32(1e4)).astype(np.float32)
    raise ValueError(kind)
