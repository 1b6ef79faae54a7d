"""Helpers shared by the GPU parity tests."""
import torch

from oracle import yamoe_oracle as O

# tolerances of the parity contract: relative L2 error of the HIP result against the oracle
REL_L2_TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2, torch.float64: 1e-13}

KEYS = ("hidden", "router_indices", "routing_weights", "gate_up_proj", "gate_up_proj_bias", "down_proj",
        "down_proj_bias")


def args(d):
    return tuple(d[k] for k in KEYS)


def to_dev(d, device):
    return {k: v.to(device) for k, v in d.items()}


def oracle_forward(d, capacity, compute_dtype=torch.float32):
    """fp32 (or fp64) oracle on the dtype-rounded inputs: the value the kernels should approximate."""
    return O.experts_capacity(*args(d), capacity, compute_dtype=compute_dtype)


def report(name, got, want, tol):
    r, m = O.rel_l2(got, want), O.max_abs(got, want)
    print("%s: rel_l2=%.3e max_abs=%.3e (tol %.0e)" % (name, r, m, tol), flush=True)
    return r
