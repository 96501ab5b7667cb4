"""Oracle (test infrastructure): flow-matching schedule used by the few-step sampler.

Follows utils/scheduler.py:106-176 (`FlowMatchScheduler`: sigma ladder with shift, add_noise)
and utils/wan_wrapper.py:172-196 (x0 = x_t - sigma_t * flow, in float64, sigma looked up by the
nearest table timestep); warped denoising list pipeline/causal_inference.py:33-35.
"""
import numpy as np


def sigma_table(num_steps=1000, shift=5.0, sigma_max=1.0, sigma_min=0.0, extra_one_step=True):
    if extra_one_step:
        sig = np.linspace(sigma_max, sigma_min, num_steps + 1, dtype=np.float64)[:-1]
    else:
        sig = np.linspace(sigma_max, sigma_min, num_steps, dtype=np.float64)
    sig = shift * sig / (1.0 + (shift - 1.0) * sig)
    return sig, sig * 1000.0            # sigmas, timesteps


def sigma_of(t, shift=5.0):
    sig, ts = sigma_table(shift=shift)
    return sig[np.argmin(np.abs(ts - t))]


def warped_steps(step_list=(1000, 750, 500, 250), shift=5.0):
    """timesteps[1000 - t] of the 1000-entry table extended by a trailing 0."""
    _, ts = sigma_table(shift=shift)
    ts = np.concatenate([ts, [0.0]])
    return [float(ts[1000 - t]) for t in step_list]
