"""Writes tests/golden/golden.npz: small known-answer cases for the five operations.

The reference (lab-cosmo/mops) ships no golden vectors; its tests draw random
inputs and compare with `reference_implementations.py`
(python/mops/tests/*.py). The expected values here are made the same way but
by code that shares nothing with the oracle or the HIP kernels:

* outputs: dense float64 formulations written with `torch.einsum` /
  `index_add_` (the definitions quoted in the docstrings below);
* gradients: `torch.autograd.grad` of those formulations against the stored
  `grad_output` (float64), i.e. torch's differentiation rules, not ours;
* second order (HPE, SAP, OPSA, the operations that have a vjp_vjp): the
  stored cotangents `grad_grad_*` are contracted with those gradients and
  differentiated once more by torch with respect to `grad_output`, A and B.

Inputs are float64 values that are exactly representable in float32
(multiples of 1/64), so the same fixture serves both precisions; expected
values are float64.

Run `python tests/golden/make_golden.py` from the repository root (CPU only).
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def grid(rng, shape):
    """Random multiples of 1/64 in [-2, 2): exact in float32 and float64."""
    return rng.integers(-128, 128, size=shape).astype(np.float64) / 64.0


def sorted_index(rng, n_out, n_in, empty_rows=()):
    allowed = np.array([v for v in range(n_out) if v not in empty_rows])
    return np.sort(rng.choice(allowed, size=n_in)).astype(np.int32)


def hpe(A, C, indices_A):
    """O[i] = sum_j C[j] * prod_k A[i, indices_A[j, k]]"""
    if indices_A.shape[1] == 0:
        return C.sum() * torch.ones(A.shape[0], dtype=A.dtype)
    return torch.prod(A[:, indices_A.long()], dim=2) @ C


def sap(A, B, C, indices_A, indices_B, indices_output, output_size):
    """O[i, indices_output[k]] += C[k] * A[i, indices_A[k]] * B[i, indices_B[k]]"""
    terms = C[None, :] * A[:, indices_A.long()] * B[:, indices_B.long()]
    out = torch.zeros(A.shape[0], output_size, dtype=A.dtype)
    return out.index_add(1, indices_output.long(), terms)


def opsa(A, B, indices_output, output_size):
    """O[indices_output[j], k, l] += A[j, k] * B[j, l]"""
    out = torch.zeros(output_size, A.shape[1], B.shape[1], dtype=A.dtype)
    return out.index_add(0, indices_output.long(), torch.einsum("jk,jl->jkl", A, B))


def opsaw(A, B, W, indices_W, indices_output):
    """O[indices_output[e], k, l] += A[e, k] * B[e, l] * W[indices_W[e], l]"""
    out = torch.zeros(W.shape[0], A.shape[1], B.shape[1], dtype=A.dtype)
    return out.index_add(0, indices_output.long(), torch.einsum("ek,el->ekl", A, B * W[indices_W.long()]))


def sasaw(A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2, output_size):
    """O[PO1[e], PO2[n], :] += C[n] * A[e, PA[n]] * B[e, :] * W[PW1[e], PW2[n], :]"""
    per_entry = (
        C[None, :, None]
        * A[:, indices_A.long()][:, :, None]
        * B[:, None, :]
        * W[indices_W_1.long()][:, indices_W_2.long(), :]
    )  # [e, n, l]
    per_edge = torch.zeros(A.shape[0], output_size, B.shape[1], dtype=A.dtype)
    per_edge = per_edge.index_add(1, indices_output_2.long(), per_entry)
    out = torch.zeros(W.shape[0], output_size, B.shape[1], dtype=A.dtype)
    return out.index_add(0, indices_output_1.long(), per_edge)


FORMULAS = {"hpe": hpe, "sap": sap, "opsa": opsa, "opsaw": opsaw, "sasaw": sasaw}
INPUTS = {
    "hpe": ["A", "C", "indices_A"],
    "sap": ["A", "B", "C", "indices_A", "indices_B", "indices_output", "output_size"],
    "opsa": ["A", "B", "indices_output", "output_size"],
    "opsaw": ["A", "B", "W", "indices_W", "indices_output"],
    "sasaw": ["A", "B", "C", "W", "indices_A", "indices_W_1", "indices_W_2", "indices_output_1",
              "indices_output_2", "output_size"],
}  # fmt: skip
DIFFERENTIABLE = {"hpe": ["A"], "sap": ["A", "B"], "opsa": ["A", "B"], "opsaw": ["A", "B", "W"],
                  "sasaw": ["A", "B", "W"]}  # fmt: skip


def cases():
    rng = np.random.default_rng(20240607)
    out = {}
    # HPE: order 3 with repeated factors, order 0, order 1
    out["hpe/order3"] = dict(A=grid(rng, (7, 5)), C=grid(rng, 11), indices_A=rng.integers(0, 5, (11, 3)).astype(np.int32))
    out["hpe/order0"] = dict(A=grid(rng, (4, 3)), C=grid(rng, 6), indices_A=np.zeros((6, 0), np.int32))
    out["hpe/order1"] = dict(A=grid(rng, (5, 4)), C=grid(rng, 9), indices_A=rng.integers(0, 4, (9, 1)).astype(np.int32))
    # SAP: sorted and unsorted output index, an output column nobody writes
    out["sap/sorted"] = dict(A=grid(rng, (9, 4)), B=grid(rng, (9, 3)), C=grid(rng, 14),
                             indices_A=rng.integers(0, 4, 14).astype(np.int32),
                             indices_B=rng.integers(0, 3, 14).astype(np.int32),
                             indices_output=np.sort(rng.choice([0, 1, 3, 4], 14)).astype(np.int32), output_size=5)
    out["sap/unsorted"] = dict(A=grid(rng, (70, 3)), B=grid(rng, (70, 2)), C=grid(rng, 8),
                               indices_A=rng.integers(0, 3, 8).astype(np.int32),
                               indices_B=rng.integers(0, 2, 8).astype(np.int32),
                               indices_output=rng.integers(0, 4, 8).astype(np.int32), output_size=4)
    # OPSA / OPSAW / SASAW: rows 1 and 4 receive nothing
    out["opsa/empty_rows"] = dict(A=grid(rng, (40, 3)), B=grid(rng, (40, 5)),
                                  indices_output=sorted_index(rng, 6, 40, (1, 4)), output_size=6)
    out["opsa/no_edges"] = dict(A=grid(rng, (0, 3)), B=grid(rng, (0, 2)),
                                indices_output=np.zeros(0, np.int32), output_size=3)
    out["opsaw/empty_rows"] = dict(A=grid(rng, (50, 2)), B=grid(rng, (50, 6)), W=grid(rng, (6, 6)),
                                   indices_W=rng.integers(0, 6, 50).astype(np.int32),
                                   indices_output=sorted_index(rng, 6, 50, (1, 4)))
    out["sasaw/empty_rows"] = dict(A=grid(rng, (45, 4)), B=grid(rng, (45, 6)), C=grid(rng, 17), W=grid(rng, (6, 3, 6)),
                                   indices_A=rng.integers(0, 4, 17).astype(np.int32),
                                   indices_W_1=rng.integers(0, 6, 45).astype(np.int32),
                                   indices_W_2=rng.integers(0, 3, 17).astype(np.int32),
                                   indices_output_1=sorted_index(rng, 6, 45, (1, 4)),
                                   indices_output_2=rng.integers(0, 5, 17).astype(np.int32), output_size=5)
    return out


def main():
    arrays = {}
    for name, case in cases().items():
        op = name.split("/")[0]
        tensors = {}
        for key in INPUTS[op]:
            value = case[key]
            if isinstance(value, np.ndarray):
                tensor = torch.from_numpy(value.copy())
                if key in DIFFERENTIABLE[op]:
                    tensor.requires_grad_(True)
                tensors[key] = tensor
            else:
                tensors[key] = value
        output = FORMULAS[op](*[tensors[key] for key in INPUTS[op]])
        rng = np.random.default_rng(sum(name.encode()) * 7919)
        grad_output = grid(rng, tuple(output.shape))
        wanted = [tensors[key] for key in DIFFERENTIABLE[op]]
        upstream = torch.from_numpy(grad_output).requires_grad_(True)
        live = output.requires_grad and output.numel() > 0 and all(t.numel() > 0 for t in wanted)
        if live:
            gradients = torch.autograd.grad(output, wanted, upstream, allow_unused=True, create_graph=True)
        else:
            gradients = [torch.zeros_like(t) for t in wanted]
        if op in ("hpe", "sap", "opsa"):
            cotangents = [grid(rng, tuple(t.shape)) for t in wanted]
            contracted = sum(
                (torch.from_numpy(c) * g).sum() for c, g in zip(cotangents, gradients) if g is not None
            )
            targets = [upstream] + wanted
            if live and isinstance(contracted, torch.Tensor) and contracted.requires_grad:
                second = torch.autograd.grad(contracted, targets, allow_unused=True)
            else:
                second = [None] * len(targets)
            second = [torch.zeros_like(t) if g is None else g.detach().clone() for t, g in zip(targets, second)]
            for g in second:
                # torch differentiates prod() through a division: what should be an exact
                # zero (second derivative of an order-1 polynomial) comes out as ~1e-16
                g[g.abs() < 1e-12] = 0.0
            for key, c in zip(DIFFERENTIABLE[op], cotangents):
                arrays[f"{name}/in/grad_grad_{key}"] = c
            arrays[f"{name}/out/grad_grad_output"] = second[0].detach().numpy()
            for key, g in zip(DIFFERENTIABLE[op], second[1:]):
                arrays[f"{name}/out/grad_{key}_2"] = g.detach().numpy()
        for key, value in case.items():
            arrays[f"{name}/in/{key}"] = np.asarray(value)
        arrays[f"{name}/in/grad_output"] = grad_output
        arrays[f"{name}/out/output"] = output.detach().numpy()
        for key, g in zip(DIFFERENTIABLE[op], gradients):
            arrays[f"{name}/out/grad_{key}"] = (torch.zeros_like(tensors[key]) if g is None else g).detach().numpy()
    np.savez_compressed(os.path.join(HERE, "golden.npz"), **arrays)
    print(f"wrote {len(arrays)} arrays for {len(cases())} cases")


if __name__ == "__main__":
    main()
