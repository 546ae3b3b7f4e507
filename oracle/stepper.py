"""Float64 restatement of Makani's model wrappers (oracle; test infrastructure only).

Follows makani/models/stepper.py:21-129 and the parts of makani/models/preprocessor.py they call (history statistics
300-322, normalisation 325-372, static features 193-199, residual rule 180-191, history feed-back 209-244) for one GPU,
as plain functions on numpy arrays; `model` is any callable [B, C_in, H, W] -> [B, C_out, H, W] on float64 arrays.
"""
import numpy as np


def history_weights(mode, n_history, decay=None):
    nh = n_history + 1
    if mode == "exponential":
        w = np.exp(-decay * np.arange(n_history, -1, -1, dtype=np.float64))
        return w / w.sum()
    if mode == "mean":
        return np.full(nh, 1.0 / nh)
    return np.ones(nh)


def history_stats(x, n_history, weights):
    """x [B, T*C, H, W] -> (mean, std) [B, C, 1, 1]: weighted over the T = n_history + 1 steps, averaged over the grid."""
    B, TC, H, W = x.shape
    T = n_history + 1
    xr = x.reshape(B, T, TC // T, H, W)
    w = weights.reshape(1, T, 1, 1, 1)
    mean = (xr * w).sum(axis=(1, 3, 4), keepdims=True) / (H * W)
    var = (np.square(xr - mean) * w).sum(axis=(1, 3, 4), keepdims=True) / (H * W)
    return mean[:, 0], np.sqrt(var[:, 0])


def single_step(model, inp, n_history=0, mode="none", decay=None, static=None, learn_residual=False, residual_scale=None, forcing=None):
    """One wrapped model call (stepper.py:27-47).  forcing: unpredicted channels [B, T, Cz, H, W] appended to every history step."""
    B, TC, H, W = inp.shape
    T = n_history + 1
    x = inp
    if forcing is not None:
        x = np.concatenate([inp.reshape(B, T, TC // T, H, W), forcing], axis=2).reshape(B, -1, H, W)
    if mode in ("none", "timediff"):
        mean, std = 0.0, 1.0
        xn = x
    else:
        mean, std = history_stats(x, n_history, history_weights(mode, n_history, decay))
        xn = (x - np.tile(mean, (1, T, 1, 1))) / np.tile(std, (1, T, 1, 1))
    if static is not None:
        xn = np.concatenate([xn, np.broadcast_to(static, (B,) + static.shape[1:])], axis=1)
    yn = model(xn)
    if mode in ("none", "timediff"):
        y = yn
    else:
        y = yn * std[:, : yn.shape[1]] + mean[:, : yn.shape[1]]
    if not learn_residual:
        return y
    if residual_scale is not None:
        y = y * residual_scale
    out = inp.reshape(B, T, TC // T, H, W).copy()
    out[:, -1] += y
    return out.reshape(B, TC, H, W)


def multi_step_train(model, inp, n_future, n_history=0, **kw):
    """Training-mode forward of the multi-step wrapper (stepper.py:60-97): predictions of n_future + 1 fed-back steps,
    concatenated along the channels."""
    B, TC, H, W = inp.shape
    T = n_history + 1
    preds, cur = [], inp
    for step in range(n_future + 1):
        pred = single_step(model, cur.copy(), n_history=n_history, **kw)
        preds.append(pred)
        if step < n_future and n_history > 0:
            cr = cur.reshape(B, T, TC // T, H, W)
            cur = np.concatenate([cr[:, 1:], pred.reshape(B, 1, -1, H, W)], axis=1).reshape(B, TC, H, W)
        else:
            cur = pred
    return np.concatenate(preds, axis=1)
