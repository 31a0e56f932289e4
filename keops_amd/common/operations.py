"""User-level reductions that are built on an internal one, and the matching output fix-up.

Same behaviour as pykeops/pykeops/common/operations.py:7-35 (preprocess) and :38-87 (postprocess),
written for torch tensors only.
"""
import torch


def preprocess(reduction_op, formula2):
    if reduction_op in ("SumSoftMaxWeight", "SoftMax"):
        # sum_j exp(f_ij - m_i) [1, g_ij] through Max_SumShiftExpWeight, divided afterwards
        return "Max_SumShiftExpWeight", "Concat(IntCst(1)," + formula2 + ")"
    if reduction_op == "LogSumExp":
        return ("Max_SumShiftExpWeight" if formula2 else "Max_SumShiftExp"), formula2
    if reduction_op == "LogSumExpWeight":
        if not formula2:
            raise ValueError("LogSumExpWeight reduction requires a weight formula (given as formula2 kwarg)")
        return "Max_SumShiftExpWeight", formula2
    return reduction_op, formula2


def postprocess(out, binding, reduction_op, nout, opt_arg, dtype):
    if reduction_op in ("SumSoftMaxWeight", "SoftMax"):
        return out[..., 2:] / out[..., 1][..., None]
    if reduction_op in ("ArgMin", "ArgMax"):
        return out.long()
    if reduction_op in ("Min_ArgMin", "MinArgMin", "Max_ArgMax", "MaxArgMax"):
        tmp = out.view(out.shape[:-1] + (2, out.shape[-1] // 2))      # (explicit sizes: a view of no rows cannot infer one)
        return tmp[..., 0, :], tmp[..., 1, :].long()
    if reduction_op == "KMin":
        out = out.view(out.shape[:-1] + (opt_arg, out.shape[-1] // opt_arg))
        return out.squeeze(-1) if out.shape[-1] == 1 else out
    if reduction_op == "ArgKMin":
        out = out.long().view(out.shape[:-1] + (opt_arg, out.shape[-1] // opt_arg))
        return out.squeeze(-1) if out.shape[-1] == 1 else out
    if reduction_op in ("KMin_ArgKMin", "KMinArgKMin"):
        tmp = out.view(out.shape[:-1] + (opt_arg, 2, out.shape[-1] // (2 * opt_arg)))
        vals, idx = tmp[..., 0, :], tmp[..., 1, :].long()
        if vals.shape[-1] == 1:
            return vals.squeeze(-1), idx.squeeze(-1)
        return vals, idx
    if reduction_op in ("LogSumExp", "LogSumExpWeight"):
        if out.shape[-1] == 2:
            return (out[..., 0] + torch.log(out[..., 1]))[..., None]
        return out[..., 0][..., None] + torch.log(out[..., 1:])
    return out


def ConjugateGradientSolver(linop, b, eps=1e-6):
    """Conjugate gradient solution of ``linop(a) = b`` for a symmetric positive definite ``linop``
    (pykeops/pykeops/common/operations.py:90-115: same iteration, same stopping rule
    ``|r|^2 < numel(b) * eps^2``)."""
    delta = b.numel() * eps ** 2
    a = 0
    r = b.clone()
    nr2 = (r ** 2).sum()
    if nr2 < delta:
        return 0 * r
    p = r.clone()
    while True:
        Mp = linop(p)
        alp = nr2 / (p * Mp).sum()
        a = a + alp * p
        r = r - alp * Mp
        nr2new = (r ** 2).sum()
        if nr2new < delta:
            break
        p = r + (nr2new / nr2) * p
        nr2 = nr2new
    return a
