"""Shared helpers for the GPU parity tests."""
import numpy as np


def rel_err(got, want):
    """|got-want| relative to max(|want|, rms(want)): the 1e-3 bar of the GEMV /
    attention parity tests is stated on this quantity.  The rms floor keeps
    rows whose true value happens to cancel to ~0 from dominating."""
    got = np.asarray(got, dtype=np.float64).ravel()
    want = np.asarray(want, dtype=np.float64).ravel()
    floor = np.sqrt(np.mean(want ** 2)) if want.size else 0.0
    return np.abs(got - want) / np.maximum(np.abs(want), max(floor, 1e-30))


def plain_rel_err(got, want):
    """|got-want| / |want| with no floor, over the elements at least as large as the vector's rms (where a plain
    relative error is meaningful in f32): the figure the floored bar is reported beside."""
    got = np.asarray(got, dtype=np.float64).ravel()
    want = np.asarray(want, dtype=np.float64).ravel()
    big = np.abs(want) >= np.sqrt(np.mean(want ** 2)) if want.size else np.zeros(0, bool)
    big &= want != 0
    return np.abs(got[big] - want[big]) / np.abs(want[big])


def assert_close(got, want, tol, what=""):
    e = rel_err(got, want)
    i = int(np.argmax(e)) if e.size else 0
    assert e.size == 0 or e[i] <= tol, f"{what}: max rel err {e[i]:.3e} at {i} (got {np.ravel(got)[i]}, want {np.ravel(want)[i]})"


def q6k_rows(w, rows, cols):
    """Q6_K bytes [rows, cols/256, 210] -> the library's row-grouped form (KSH_Q6K_ROWS): per row all ql, then all
    qh, all scales, all d, zero padding to 16 bytes.  The definition the device repacker is checked against."""
    b = np.asarray(w, dtype=np.uint8).reshape(rows, cols // 256, 210)
    pad = -(cols // 256 * 210) % 16                 # rows are padded to 16 bytes (1536 columns: 1260 -> 1264)
    return np.concatenate([b[:, :, :128].reshape(rows, -1), b[:, :, 128:192].reshape(rows, -1),
                           b[:, :, 192:208].reshape(rows, -1), b[:, :, 208:].reshape(rows, -1),
                           np.zeros((rows, pad), np.uint8)], axis=1).reshape(-1)
