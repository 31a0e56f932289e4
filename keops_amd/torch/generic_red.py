"""Genred: the user-level generic reduction on torch tensors, with autograd.

Same constructor / call signatures, formula assembly and gradient recursion as
pykeops/pykeops/torch/generic/generic_red.py (Genred :422-695, GenredAutograd_base :72-259):
a gradient is another Genred whose formula is
``Grad_WithSavedForward(<formula>, Var(pos,dim,cat), Var(nargs,dimout,tagIJ), Var(nargs+1,dimout,tagIJ))``.
Tensors must live on a HIP device; the computation runs in libkeops_hip.
"""
import copy
import warnings

import torch

from ..common.get_options import get_tag_backend
from ..common.operations import postprocess, preprocess
from ..common.parse_type import axis2cat, complete_aliases, get_optional_flags, get_sizes, get_type
from ..keops_io import keops_binder


class Genred_parameters:
    pass


_NO_AUTODIFF = (
    "Min_ArgMin_Reduction", "Min_Reduction", "Max_ArgMax_Reduction", "Max_Reduction", "KMin_ArgKMin_Reduction",
    "KMin_Reduction",
)


def check_AD_supported(formula):
    for red in _NO_AUTODIFF:
        if formula.startswith(red):
            raise NotImplementedError(
                f"As of today, KeOps does not support autodiff through the {red} reduction. Consider extracting "
                "the relevant integer indices with a '.argmin()', '.argmax()' or '.argKmin()' reduction before "
                "using PyTorch advanced indexing to create a fully-differentiable tensor."
            )


def set_device(tagCPUGPU, tagHostDevice, device_id_request, *args):
    device_args = args[0].device
    if tagCPUGPU == 1 and tagHostDevice == 1:
        for a in args[1:]:
            if a.device.index != device_args.index:
                raise ValueError("[KeOps] Input arrays must be all located on the same device.")
    if device_id_request == -1:
        device_id = device_args.index if device_args.index is not None else 0
    else:
        device_id = device_id_request
        if device_args.index is not None and device_args.index != device_id:
            raise ValueError("[KeOps] Gpu device id of arrays is different from device id requested for computation.")
    return device_id, device_args


class GenredAutograd_base:
    @staticmethod
    def _forward(params, *args):
        result, dimout, tagIJ = GenredAutograd_base._launch(params, *args)
        return result, torch.tensor([dimout, tagIJ])

    @staticmethod
    def _launch(params, *args):
        params.optional_flags["multVar_highdim"] = (
            1 if isinstance(params.rec_multVar_highdim, int) and not isinstance(params.rec_multVar_highdim, bool)
            or params.rec_multVar_highdim else 0
        )
        tagCPUGPU, tag1D2D, tagHostDevice = get_tag_backend(params.backend, args)
        # where the data lives decides what kind of pointers the library receives, whatever the backend string says
        tagHostDevice = 1 if all(a.is_cuda for a in args) else 0
        # (get_tag_backend has rejected arguments that are partly on the host and partly on a GPU; the output buffer a
        # caller hands in must live where the arguments live, as in the reference)
        if params.out is not None and bool(params.out.is_cuda) != bool(tagHostDevice):
            raise ValueError("[KeOps] Input arrays must be all located on the same device.")
        nbatchdims = max(len(a.shape) for a in args) - 2
        use_ranges = nbatchdims > 0 or params.ranges is not None
        device_id, device_args = set_device(tagCPUGPU, tagHostDevice, params.device_id_request, *args)
        nout = params.nx if params.axis == 1 else params.ny
        batch = None
        if nbatchdims > 0 and params.ranges is None:
            nbatches = 1
            for d in range(nbatchdims):
                nbatches *= max(a.shape[d] if a.dim() == nbatchdims + 2 else 1 for a in args)
            shape = tuple(max(a.shape[d] if a.dim() == nbatchdims + 2 else 1 for a in args) for d in range(nbatchdims))
            # (every tensor variable carries every batch dimension in full: many small batches can be served as row ranges)
            full = all(a.dim() != nbatchdims + 2 or tuple(a.shape[:nbatchdims]) == shape for a in args)
            batch = (nbatches, params.nx, params.ny, full)
        elif nbatchdims == 0 and params.ranges is not None:
            batch = (0, params.nx, params.ny)  # block-sparse ranges, no batch dimensions

        def binder_for(tag_hd):
            return keops_binder["hip"](
                tagCPUGPU, tag1D2D, tag_hd, use_ranges, device_id, params.formula, params.aliases, len(args),
                params.dtype, "torch", params.optional_flags, nx=nout, ny=params.nx + params.ny - nout, batch=batch,
            ).import_module()

        host_out, staged, myconv = None, False, None
        if tagCPUGPU == 1 and tagHostDevice == 0:
            # host-resident tensors with a GPU backend: the library copies them to the device itself
            # (tagHostDevice = 0, the reference's load_args_FromHost, keops_nvrtc.cpp:46-73) ...
            if not torch.cuda.is_available():
                raise ValueError("[KeOps] the HIP backend needs a GPU: none is visible to torch")
            myconv = binder_for(0)
            if myconv.plan is not None or params.dtype == "float16":
                # ... except for reductions that the binding layer evaluates as several launches combined with
                # torch operations on the device, and for half-precision data (use_half takes device pointers):
                # those are staged here
                dev = torch.device("cuda", device_id)
                args = tuple(a.to(dev) for a in args)
                if params.ranges:
                    params = copy.copy(params)
                    params.ranges = tuple(r.to(dev) for r in params.ranges)
                if params.out is not None:
                    params = copy.copy(params)
                    host_out, params.out = params.out, None
                tagHostDevice, device_args, staged, myconv = 1, dev, True, None
            elif params.ranges:
                params = copy.copy(params)
                params.ranges = tuple(r.cpu() for r in params.ranges)
        if myconv is None:
            myconv = binder_for(tagHostDevice)
        if not all(a.is_contiguous() for a in args):
            warnings.warn(
                "[KeOps] at least one of the input tensors is not contiguous. "
                "Consider using contiguous data arrays to avoid unnecessary copies."
            )
            args = tuple(a.contiguous() for a in args)
        if params.ranges:
            # the kernels read the ranges where they read the data (keops_nvrtc.cpp:190-208)
            rdev = device_args if tagHostDevice == 1 else torch.device("cpu")
            params.ranges = tuple(r.to(device=rdev, memory_format=torch.contiguous_format, dtype=torch.int64) for r in params.ranges)
        result = myconv.genred_pytorch(device_args, params.ranges, params.nx, params.ny, nbatchdims, params.out, *args)
        if host_out is not None:
            host_out.copy_(result.view(host_out.shape))
            result = host_out
        elif staged:
            result = result.cpu()
        return result, myconv.dimout, myconv.tagIJ

    @staticmethod
    def _setup_context(ctx, inputs, outputs):
        params, *args = inputs
        result, info = outputs
        ctx.mark_non_differentiable(info)
        ctx.params = params
        ctx.dimout, ctx.tagIJ = int(info[0]), int(info[1])
        ctx.save_for_backward(*args, result)
        ctx.save_for_forward(*args, result)

    @staticmethod
    def _backward(ctx, G, _):
        params, dimout, tagIJ = ctx.params, ctx.dimout, ctx.tagIJ
        args = ctx.saved_tensors[:-1]
        nargs = len(args)
        result = ctx.saved_tensors[-1].detach()
        check_AD_supported(params.formula)
        eta = f"Var({nargs},{dimout},{tagIJ})"          # incoming gradient, shaped like the output
        resvar = f"Var({nargs + 1},{dimout},{tagIJ})"   # saved forward result
        G = G.contiguous()
        grads = []
        for var_ind, (sig, arg_ind) in enumerate(zip(params.aliases, args)):
            if not ctx.needs_input_grad[var_ind + 1]:
                grads.append(None)
                continue
            _, cat, dim, pos = get_type(sig, position_in_list=var_ind)
            var = f"Var({pos},{dim},{cat})"
            params_g = copy.copy(params)
            params_g.formula = f"Grad_WithSavedForward({params.formula},{var},{eta},{resvar})"
            params_g.aliases = params.aliases + [eta, resvar]
            params_g.out = None
            if not isinstance(params.rec_multVar_highdim, bool) and pos == params.rec_multVar_highdim:
                params_g.rec_multVar_highdim = nargs
            else:
                params_g.rec_multVar_highdim = None
            if cat == 2:
                # gradient wrt a parameter: the reduction runs over j, the sum over i is done here
                params_g.axis = 1
            else:
                params_g.axis = 1 - cat
            grad = GenredAutograd_fun(params_g, *args, G, result)
            if cat == 2:
                grad = (1.0 * grad).sum(-2)
                collapse = tuple(k for k, (x, y) in enumerate(zip(arg_ind.shape[:-1], grad.shape[:-1])) if x < y)
            else:
                # adjoint of batch broadcasting: sum over the batch dimensions that were of size 1
                collapse = tuple(k for k, (x, y) in enumerate(zip(arg_ind.shape[:-2], grad.shape[:-2])) if x < y)
            if collapse:
                grad = (1.0 * grad).sum(collapse, keepdim=True)
            grads.append(grad.reshape(arg_ind.shape))
        return (None, *grads)


def _jvp(ctx, *tangents):
    """Forward-mode rule (generic_red.py:318-380): the output tangent is the sum over the inputs that carry
    a tangent of Genred("Diff_WithSavedForward(F, v, eta, result)") evaluated at (args, tangent, result)."""
    params, dimout, tagIJ = ctx.params, ctx.dimout, ctx.tagIJ
    args = ctx.saved_tensors[:-1]
    nargs = len(args)
    result = ctx.saved_tensors[-1].detach()
    check_AD_supported(params.formula)
    resvar = f"Var({nargs + 1},{dimout},{tagIJ})"
    out = 0
    for var_ind, sig in enumerate(params.aliases):
        u = tangents[var_ind + 1]
        if u is None:
            continue
        _, cat, dim, pos = get_type(sig, position_in_list=var_ind)
        eta = f"Var({nargs},{dim},{cat})"
        params_d = copy.copy(params)
        params_d.formula = f"Diff_WithSavedForward({params.formula},Var({pos},{dim},{cat}),{eta},{resvar})"
        params_d.aliases = params.aliases + [eta, resvar]
        params_d.out = None
        params_d.rec_multVar_highdim = None
        out = out + GenredAutograd_fun(params_d, *args, u.contiguous(), result)
    return out, None


class GenredAutograd(torch.autograd.Function):
    """Entry point to the torch autograd engine (generic_red.py:262-302)."""

    @staticmethod
    def jvp(ctx, *tangents):
        return _jvp(ctx, *tangents)

    @staticmethod
    def vmap(info, in_dims, params, *args):
        # the vmapped axis becomes a leading batch dimension (generic_red.py:304-316); arguments that are
        # not vmapped get a batch dimension of size 1, which broadcasts
        args = [a[None, ...] if d is None else a.movedim(d, 0).contiguous() for a, d in zip(args, in_dims[1:])]
        p = copy.copy(params)
        p.out = None
        return GenredAutograd.apply(p, *args), (0, None)

    @staticmethod
    def forward(*inputs):
        return GenredAutograd_base._forward(*inputs)

    @staticmethod
    def setup_context(ctx, inputs, outputs):
        GenredAutograd_base._setup_context(ctx, inputs, outputs)

    @staticmethod
    def backward(ctx, G, _):
        return GenredAutograd_base._backward(ctx, G, _)


def _nothing_to_differentiate(args):
    """No argument asks for a gradient, no forward-mode level and no function transform (vmap, grad, jvp) is active."""
    if torch._C._functorch.peek_interpreter_stack() is not None or torch.autograd.forward_ad._current_level >= 0:
        return False
    return not (torch.is_grad_enabled() and any(a.requires_grad for a in args))


def GenredAutograd_fun(params, *args):
    # the autograd machinery around a launch (argument binding, context, saved tensors) costs as much as a small
    # launch itself: when there is nothing to differentiate the result is the same without it
    if _nothing_to_differentiate(args):
        return GenredAutograd_base._launch(params, *args)[0]
    return GenredAutograd.apply(params, *args)[0]


class Genred:
    r"""Generic map-reduce operation ``out_i = Reduction_j F(x_i, y_j, p)`` on torch tensors.

    Example:
        >>> my_conv = Genred('Exp(-SqNorm2(x - y))', ['x = Vi(3)', 'y = Vj(3)'], reduction_op='Sum', axis=1)
        >>> a = my_conv(x, y)   # x: (M,3), y: (N,3) device tensors -> a: (M,1)
    """

    def __init__(self, formula, aliases, reduction_op="Sum", axis=0, dtype=None, opt_arg=None, formula2=None,
                 cuda_type=None, dtype_acc="auto", use_double_acc=False, sum_scheme="auto", enable_chunks=True,
                 rec_multVar_highdim=False, use_fast_math=True):
        if dtype:
            warnings.warn("[KeOps] keyword argument dtype in Genred is deprecated ; argument is ignored.")
        if cuda_type:
            warnings.warn("[KeOps] keyword argument cuda_type in Genred is deprecated ; argument is ignored.")
        self.reduction_op = reduction_op
        reduction_op_internal, formula2 = preprocess(reduction_op, formula2)
        self.optional_flags = get_optional_flags(
            reduction_op_internal, dtype_acc, use_double_acc, sum_scheme, enable_chunks, use_fast_math
        )
        str_opt_arg = f",{opt_arg}" if opt_arg else ""
        str_formula2 = f",{formula2}" if formula2 else ""
        self.formula = f"{reduction_op_internal}_Reduction({formula}{str_opt_arg},{axis2cat(axis)}{str_formula2})"
        self.aliases = complete_aliases(self.formula, list(aliases))
        self.nargs = len(self.aliases)
        self.axis = axis
        self.opt_arg = opt_arg
        self.rec_multVar_highdim = rec_multVar_highdim

    def __call__(self, *args, backend="auto", device_id=-1, ranges=None, out=None):
        if len(args) != self.nargs:
            raise ValueError(
                f"Invalid number of arguments in call to Genred (should be {self.nargs} and got {len(args)})."
            )
        dtype = str(args[0].dtype).split(".")[1]
        nx, ny = get_sizes(self.aliases, *args)
        nout, nred = (nx, ny) if self.axis == 1 else (ny, nx)
        if "Arg" in self.reduction_op and nred > 1.6e7 and dtype == "float32":
            raise ValueError(
                "size of input array is too large for Arg type reduction with single precision. Use double precision."
            )
        params = Genred_parameters()
        params.formula, params.aliases = self.formula, self.aliases
        params.backend, params.dtype = backend, dtype
        params.device_id_request, params.ranges = device_id, ranges
        params.optional_flags = dict(self.optional_flags)
        params.rec_multVar_highdim = self.rec_multVar_highdim
        params.nx, params.ny, params.axis, params.out = nx, ny, self.axis, out
        out = GenredAutograd_fun(params, *args)
        return postprocess(out, "torch", self.reduction_op, nout, self.opt_arg, dtype)
