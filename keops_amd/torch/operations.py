"""KernelSolve: conjugate-gradient solver for ``(alpha Id + K_xx) a = b`` built on the generic reduction.

Same constructor / call signatures, iteration and gradient as pykeops/pykeops/torch/operations.py
(KernelSolveAutograd :23-165, KernelSolve :168-430): the forward pass runs the conjugate gradient
with the kernel product evaluated by the map-reduce kernels; the backward pass solves the adjoint
system once and differentiates the formula with ``Grad_WithSavedForward`` through Genred.
"""
import copy
import warnings

import torch

from ..common.operations import ConjugateGradientSolver
from ..common.parse_type import axis2cat, complete_aliases, get_optional_flags, get_sizes, get_type
from .generic_red import Genred_parameters, GenredAutograd_base, GenredAutograd_fun


class KernelSolveAutograd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, params, *args):
        varinv = args[params.varinvpos]

        def linop(var):
            newargs = args[: params.varinvpos] + (var.contiguous(),) + args[params.varinvpos + 1:]
            res = GenredAutograd_base._forward(params, *newargs)[0]
            if params.alpha:
                res = res + params.alpha * var
            return res

        with torch.no_grad():
            result = ConjugateGradientSolver(linop, varinv.detach(), params.eps)
        ctx.params = params
        ctx.save_for_backward(*args, result)
        return result

    @staticmethod
    def backward(ctx, G):
        params = ctx.params
        args = ctx.saved_tensors[:-1]
        nargs = len(args)
        result = ctx.saved_tensors[-1]
        dimout, tagIJ = G.shape[-1], params.tagIJ  # the gradient has the shape of the output
        eta = f"Var({nargs},{dimout},{tagIJ})"
        resvar = f"Var({nargs + 1},{dimout},{tagIJ})"
        newargs = args[: params.varinvpos] + (G.contiguous(),) + args[params.varinvpos + 1:]
        KinvG = KernelSolveAutograd.apply(params, *newargs)
        grads = []
        for var_ind, sig in enumerate(params.aliases):
            if not ctx.needs_input_grad[var_ind + 1]:
                grads.append(None)
                continue
            if var_ind == params.varinvpos:
                grads.append(KinvG)
                continue
            _, cat, dim, pos = get_type(sig, position_in_list=var_ind)
            var = f"Var({pos},{dim},{cat})"
            params_g = copy.copy(params)
            params_g.formula = f"Grad_WithSavedForward({params.formula},{var},{eta},{resvar})"
            params_g.aliases = params.aliases + [eta, resvar]
            params_g.out = None
            params_g.rec_multVar_highdim = None
            params_g.axis = 1 if cat == 2 else 1 - cat
            args_g = args[: params.varinvpos] + (result,) + args[params.varinvpos + 1:] + (-KinvG, result)
            grad = GenredAutograd_fun(params_g, *args_g)
            if cat == 2:
                grad = (1.0 * grad).sum(-2)
            grads.append(grad.reshape(args[var_ind].shape))
        return (None, *grads)


class KernelSolve:
    r"""Conjugate gradient solver ``a = (alpha Id + K_xx)^{-1} b`` for a symmetric positive definite
    kernel operator given by a formula that is linear in the variable ``varinvalias``.

    Example:
        >>> formula = "Exp(-Norm2(x - y)) * a"
        >>> aliases = ["x = Vi(3)", "y = Vj(3)", "a = Vj(2)"]
        >>> K_inv = KernelSolve(formula, aliases, "a", axis=1)
        >>> a = K_inv(x, x, b, alpha=0.1)     # x: (N,3), b: (N,2) device tensors
    """

    def __init__(self, formula, aliases, varinvalias, axis=0, dtype_acc="auto", use_double_acc=False, sum_scheme="auto",
                 enable_chunks=True, rec_multVar_highdim=None, dtype=None, cuda_type=None, use_fast_math=True):
        if dtype:
            warnings.warn("[KeOps] keyword argument dtype in KernelSolve is deprecated ; argument is ignored.")
        if cuda_type:
            warnings.warn("[KeOps] keyword argument cuda_type in KernelSolve is deprecated ; argument is ignored.")
        self.reduction_op = "Sum"
        self.optional_flags = get_optional_flags(self.reduction_op, dtype_acc, use_double_acc, sum_scheme, enable_chunks,
                                                 use_fast_math)
        self.formula = f"{self.reduction_op}_Reduction({formula},{axis2cat(axis)})"
        self.aliases = complete_aliases(formula, list(aliases))
        if varinvalias[:4] == "Var(":
            varinvpos = int(varinvalias[4: varinvalias.find(",")])
        else:
            names = [s[: s.find("=")].strip() for s in self.aliases]
            varinvpos = names.index(varinvalias)
        self.varinvpos = varinvpos
        self.rec_multVar_highdim = rec_multVar_highdim
        self.axis = axis

    def __call__(self, *args, backend="auto", device_id=-1, alpha=1e-10, eps=1e-6, ranges=None):
        dtype = str(args[0].dtype).split(".")[1]
        nx, ny = get_sizes(self.aliases, *args)
        params = Genred_parameters()
        params.formula, params.aliases = self.formula, self.aliases
        params.varinvpos, params.alpha, params.eps = self.varinvpos, alpha, eps
        params.backend, params.dtype = backend, dtype
        params.device_id_request, params.ranges = device_id, ranges
        params.optional_flags = dict(self.optional_flags)
        params.rec_multVar_highdim = self.rec_multVar_highdim
        params.nx, params.ny, params.axis, params.out = nx, ny, self.axis, None
        params.tagIJ = axis2cat(self.axis)  # category of the output (and of the unknown's right-hand side)
        return KernelSolveAutograd.apply(params, *args)
