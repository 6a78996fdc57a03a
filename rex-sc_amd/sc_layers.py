"""SC layers: counterparts of the reference's utils_class.py (Conv2d_Add_Partial :14-86, Linear_Or :183-208)."""
import os

import torch
import torch.nn as nn

import _ops
import sc_functional as utils_f


class Conv2d_Add_Partial(nn.Conv2d):
    """SC Conv2d with OR-n partial binary accumulation.

    Keyword arguments beyond nn.Conv2d's (defaults as utils_class.py:19-34): approx, forward
    ('or_2'), generator ('lfsr'), err (stream length 2**err, 6), load_unit (8), load_wait_w (1),
    load_wait_a (1), prec_out (24), sync (1), prec (7), split_output, order (5), scale_offset.
    Buffers weight_flag, prune, bias_coef, std_coef keep the reference's names so state_dicts
    interchange.  dilation and bias are accepted by nn.Conv2d but ignored by the SC path, groups are
    a Python loop -- all as in the reference.
    """

    def __init__(self, *kargs, **kwargs):
        self.run_args = {}
        for key, default in (("approx", False), ("forward", "or_2"), ("generator", "lfsr"), ("err", 6),
                             ("load_unit", 8), ("load_wait_w", 1), ("load_wait_a", 1), ("prec_out", 24),
                             ("sync", 1), ("prec", 7), ("split_output", False), ("order", 5), ("scale_offset", 0)):
            utils_f.setdict_default(self.run_args, kwargs, key, default)
        self.run_args["bit_length"] = 2 ** self.run_args["err"]
        super(Conv2d_Add_Partial, self).__init__(*kargs, **kwargs)
        self.register_buffer("weight_flag", self.weight.data.clone())
        self.register_buffer("prune", torch.tensor([0.]))
        self.register_buffer("bias_coef", torch.zeros(self.run_args["order"] + 1))
        self.register_buffer("std_coef", torch.zeros(self.run_args["order"] + 1))
        self._weight_streams = _ops.WeightStreamCache()  # not a buffer: derived data, never part of a state_dict

    def train(self, mode=True):
        if mode:  # training regenerates the streams on every call: give the kept ones back
            self._weight_streams.clear()
        return super(Conv2d_Add_Partial, self).train(mode)

    def _load_from_state_dict(self, *args, **kwargs):
        self._weight_streams.clear()
        return super(Conv2d_Add_Partial, self)._load_from_state_dict(*args, **kwargs)

    def _fn_args(self):
        keys = ("bit_length", "generator", "forward", "load_unit", "load_wait_w", "split_output", "order", "sync")
        return {k: self.run_args[k] for k in keys}

    def forward(self, input):
        if os.environ.get("Weight_Prec", "-1") != "-1":
            weight_prec = int(os.environ.get("Weight_Prec"))
        else:
            weight_prec = self.run_args["prec"]
        if self.groups == 1 and self.run_args["sync"] == 1 and not torch.is_grad_enabled():
            # evaluation: SC forward alone, quantisation folded into the generators, weight streams kept between
            # calls and regenerated on the device when the weights' values have changed, by whatever route
            # (REXSC_WEIGHT_STREAM_CACHE=0 regenerates them on every call)
            cache = self._weight_streams if os.environ.get("REXSC_WEIGHT_STREAM_CACHE", "1") != "0" else None
            out = utils_f.conv2d_sc_inference(input, self.weight, self.padding, self.stride, self.run_args["prec"], weight_prec,
                                              weight_stream_cache=cache, **self._fn_args())
            if out is not None:
                return out
        input = utils_f.QuantizeGrad.apply(input, self.run_args["prec"])
        g_in = input.size(1) // self.groups
        g_wgt = self.weight.size(0) // self.groups
        weight = utils_f.QuantizeGrad.apply(self.weight, weight_prec)
        out_list = []
        for g in range(self.groups):
            x_g = input if self.groups == 1 else input[:, g * g_in:(g + 1) * g_in]
            w_g = weight if self.groups == 1 else weight[g * g_wgt:(g + 1) * g_wgt]
            args = self._fn_args()
            args["bias_coef"] = self.bias_coef
            args["std_coef"] = self.std_coef
            if self.run_args["sync"] == 2:
                out, self.bias_coef, self.std_coef = utils_f.conv2d_generic(x_g, w_g, padding=self.padding,
                                                                            stride=self.stride, **args)
            else:
                out = utils_f.conv2d_generic(x_g, w_g, padding=self.padding, stride=self.stride, **args)
            out_list.append(out)
        if self.groups == 1:
            return out_list[0]
        out = torch.stack(out_list, dim=2)
        return out.reshape(input.size(0), -1, out.size(3), out.size(4))


class Linear_Or(nn.Linear):
    """SC linear layer (OR accumulation over the input features).

    Default: the extension kernels' semantics (sc_matmul.cpp:576-676) with the keyword arguments of
    Conv2d_Add_Partial (forward 'or_2', generator 'lfsr', err 6, load_unit, load_wait_w, sync, prec 7).
    legacy=True: the reference's own Linear_Or (utils_class.py:183-208), which runs the legacy simulation
    `linear_generic` (seeds 67/37/0, full OR accumulation): forward(input, prec=7, err=7, generator='lfsr')
    quantises the input in place and the weight through QuantizeGrad, then calls
    linear_generic(input, weight, bit_length=2**err, forward='full_or', generator=generator)."""

    def __init__(self, *kargs, **kwargs):
        self.run_args = {}
        self.legacy = bool(kwargs.pop("legacy", False))
        for key, default in (("forward", "or_2"), ("generator", "lfsr"), ("err", 6), ("load_unit", 8),
                             ("load_wait_w", 1), ("sync", 1), ("prec", 7)):
            utils_f.setdict_default(self.run_args, kwargs, key, default)
        self.run_args["bit_length"] = 2 ** self.run_args["err"]
        super(Linear_Or, self).__init__(*kargs, **kwargs)
        self.register_buffer("weight_flag", self.weight.data.clone())
        self._weight_streams = _ops.WeightStreamCache()

    def train(self, mode=True):
        if mode:
            self._weight_streams.clear()
        return super(Linear_Or, self).train(mode)

    def _load_from_state_dict(self, *args, **kwargs):
        self._weight_streams.clear()
        return super(Linear_Or, self)._load_from_state_dict(*args, **kwargs)

    def forward(self, input, prec=7, err=7, generator="lfsr"):
        if self.legacy:
            input.data = utils_f.quantize(input.data, prec=prec)
            weight = utils_f.QuantizeGrad.apply(self.weight, prec)
            return utils_f.linear_generic(input, weight, bit_length=2 ** err, forward="full_or", generator=generator)
        keys = ("bit_length", "forward", "generator", "load_unit", "load_wait_w", "sync")
        if self.run_args["sync"] == 1 and not torch.is_grad_enabled() and input.is_cuda:
            # evaluation: the weight bitstreams are kept between calls and regenerated on the device when the
            # weights' values have changed (REXSC_WEIGHT_STREAM_CACHE=0 regenerates them on every call)
            cache = self._weight_streams if os.environ.get("REXSC_WEIGHT_STREAM_CACHE", "1") != "0" else None
            return utils_f.linear_sc_inference(input, self.weight, self.run_args["prec"], weight_stream_cache=cache,
                                               **{k: self.run_args[k] for k in keys})
        input = utils_f.QuantizeGrad.apply(input, self.run_args["prec"])
        weight = utils_f.QuantizeGrad.apply(self.weight, self.run_args["prec"])
        return utils_f.linear_generic_sc(input, weight, **{k: self.run_args[k] for k in keys})
