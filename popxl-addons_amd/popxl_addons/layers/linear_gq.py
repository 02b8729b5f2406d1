"""Group-quantised linear layer on the GPU (eager), with the constructor, variable names and
shapes, matmul orientation and `torch_mapping` of the reference's
popxl_addons/layers/linear_gq.py:19-136."""
from typing import Optional

import numpy as np

from popxl_addons import _gq_hip
from popxl_addons.ops.group_quantize_decompress import (
    group_quantize_compress,
    group_quantize_compress_numpy,
)
from popxl_addons.utils import NamedTensors, Variable, WeightsDict, _numpy_dtype_of


class GroupSizeError(ValueError, ZeroDivisionError):
    """group_size was left at 0 (the constructor default); the reference fails with a
    ZeroDivisionError at build time in that case (linear_gq.py:73)."""


class LinearGQ:
    def __init__(
        self,
        out_features: int,
        bias: bool = True,
        replica_grouping=None,
        group_size: int = 0,
        dim: int = -1,
    ):
        """
        Group Quantised Linear layer.

        Stores quantised weights as three variables:
            weight_compressed: packed integer ids, four 4-bit integers per uint16 element
            weight_decompression_scale: float16 scale per group
            weight_decompression_bias: float16 bias per group
        and an optional additive `bias`.  Variables are zero-initialised on the first build;
        overwrite them with `load_weights` (see `torch_mapping`).

        Arguments:
        - out_features (int): output dimension of layer
        - bias (bool): add a bias term (default True)
        - replica_grouping: must be None (single GPU, no variable sharding)
        - group_size (int): values per (scale, bias) pair; must be set to a positive multiple of 4
        - dim (int): dimension of the [in, out] weight matrix that is grouped.
                     0: groups run along the input features;
                     1 or -1: groups run along the output features.
                     Both layouts run fused dequant-matmul kernels.
        """
        if replica_grouping is not None:
            raise NotImplementedError("LinearGQ here runs on one GPU: replica_grouping must be None")
        self.out_features = out_features
        self.bias = bias
        self.replica_grouping = replica_grouping
        self.group_size = group_size
        self.dim = dim
        self.variables: Optional[NamedTensors] = None
        self._decode_copy = None  # the weight in the streaming layout of its dim, once prepack_for_decode has made it

    # ----------------------------------------------------------------------------- variables

    def _variable_shapes(self, in_features):
        # linear_gq.py:59-97
        if self.group_size == 0:
            raise GroupSizeError("LinearGQ: group_size is 0; set it to a positive multiple of 4")
        if self.dim in [1, -1]:
            compressed_dim, uncompressed_dim = self.out_features, in_features
        elif self.dim == 0:
            uncompressed_dim, compressed_dim = self.out_features, in_features
        else:
            raise ValueError(f"LinearGQ: dim must be 0, 1 or -1, got {self.dim}")
        n_groups = compressed_dim // self.group_size
        return (uncompressed_dim, n_groups, self.group_size // 4), (uncompressed_dim, n_groups, 1)

    def init_variables(self, in_features, dtype, device):
        import torch

        packed_shape, stat_shape = self._variable_shapes(in_features)
        named = NamedTensors(
            weight_compressed=Variable("weight_compressed", torch.zeros(packed_shape, dtype=torch.uint16, device=device)),
            weight_decompression_scale=Variable(
                "weight_decompression_scale", torch.zeros(stat_shape, dtype=dtype, device=device)
            ),
            weight_decompression_bias=Variable(
                "weight_decompression_bias", torch.zeros(stat_shape, dtype=dtype, device=device)
            ),
        )
        if self.bias:
            named.insert("bias", Variable("bias", torch.zeros((self.out_features,), dtype=dtype, device=device)))
        self.variables = named
        return named

    def load_weights(self, weights):
        """Copy a WeightsDict (or a callable producing one from the variables) into the variables."""
        import torch

        if callable(weights):
            weights = weights(self.variables)
        for var, value in weights.items():
            var.data.copy_(torch.from_numpy(np.ascontiguousarray(value)).to(var.data.device))
        if self._decode_copy is not None:  # (a derived copy of the variables: make it again)
            self._decode_copy = None
            self.prepack_for_decode()

    # --------------------------------------------------------------------------------- build

    def build(self, x, activation=None):
        """y = x @ decompress(weight) (+ bias), linear_gq.py:99-109.  x: float16 [..., in] on the GPU.

        activation (None, "relu", "gelu_tanh") is an addition to the reference's signature: the
        epilogue is fused into the kernel."""
        import torch

        act = _gq_hip.activation_code(activation)

        if not x.is_cuda:
            raise RuntimeError("LinearGQ runs on the GPU only: move x to a HIP device")
        in_features = x.shape[-1]
        if self.variables is None:
            self.init_variables(in_features, x.dtype, x.device)
        v = self.variables
        if x.dtype != torch.float16 or v.weight_decompression_scale.dtype != torch.float16:
            raise TypeError("LinearGQ: only float16 activations and float16 scale/bias are supported")
        packed_shape, _ = self._variable_shapes(in_features)
        if v.weight_compressed.shape != packed_shape:
            raise ValueError(f"LinearGQ: x has {in_features} features but weight_compressed is {v.weight_compressed.shape}")
        b = v.bias.data if self.bias else None

        # A decode batch that is a column slice of a wider matrix (part of the output of fused projections, say)
        # is read where it lies, its rows a stride apart; anything else is gathered into a contiguous x.
        x_row_stride = 0
        takes_stride = self.dim == 0 or (self._decode_copy is not None and x.data_ptr() % 16 == 0 and x.dim() == 2
                                         and x.stride(0) % 8 == 0)
        if (takes_stride and x.dim() == 2 and not x.is_contiguous() and x.stride(1) == 1 and x.stride(0) >= in_features
                and 0 < x.shape[0] <= 16):
            x2, x_row_stride = x, x.stride(0)
        else:
            x2 = x.reshape(-1, in_features).contiguous()
        m_rows = x2.shape[0]
        with torch.cuda.device(x.device):
            y = torch.empty((m_rows, self.out_features), dtype=torch.float16, device=x.device)
            args = (
                x2.data_ptr(),
                m_rows,
                v.weight_compressed.data.data_ptr(),
                v.weight_decompression_scale.data.data_ptr(),
                v.weight_decompression_bias.data.data_ptr(),
                0 if b is None else b.data_ptr(),
                y.data_ptr(),
                self.out_features,
                in_features,
                self.group_size,
                act,
            )
            stream = torch.cuda.current_stream(x.device).cuda_stream
            if x_row_stride and self.dim == 0:
                blob = 0 if self._decode_copy is None else self._decode_copy.blob.data_ptr()
                _gq_hip.call("gq_linear_p_strided_f16", args[0], x_row_stride, *args[1:5], blob, *args[5:], stream)
            elif self.dim == 0:
                # (few output tiles: several workgroups divide the input features of a tile through a workspace)
                need = _gq_hip.load().gq_gemm_workspace_bytes(m_rows, self.out_features, in_features, self.group_size)
                ws = _gq_hip.linear_kn_workspace(x.device, need) if need > 0 else None
                # (with the derived copy the pipelined GEMM kernel reads that; everything else reads the variables)
                blob = 0 if self._decode_copy is None else self._decode_copy.blob.data_ptr()
                _gq_hip.call("gq_linear_p_act_f16", *args[:5], blob, *args[5:], 0 if ws is None else ws.data_ptr(),
                             0 if ws is None else ws.numel(), stream)
            elif self._decode_copy is not None:
                # groups along the output features, the derived copy is there (x2 contiguous, or rows a stride apart)
                _gq_hip.linear_knp(x2, self._decode_copy, b, act, y)
            else:
                # groups along the output features: weight rows are input features
                need = _gq_hip.load().gq_linear_kn_workspace_bytes(m_rows, self.out_features, in_features, self.group_size)
                ws = _gq_hip.linear_kn_workspace(x.device, need) if need > 0 else None
                _gq_hip.call("gq_linear_kn_act_f16", *args, 0 if ws is None else ws.data_ptr(),
                             0 if ws is None else ws.numel(), stream)
        return y.reshape(*x.shape[:-1], self.out_features)

    __call__ = build

    # ------------------------------------------------------------------------------- fusion

    @classmethod
    def fuse(cls, layers):
        """One layer computing the concatenated outputs of `layers` (e.g. the Q, K and V projections
        of a decoder block, which read the same activations): y = cat([l(x) for l in layers], -1) in
        a single kernel pass over x.  The variables of the layers stack along their first axis for
        dim=0 (weight rows are output features) and along the group axis for dim=-1 / 1 (weight rows
        are input features); all layers must agree in dim, group_size, bias and input width.  The
        new layer owns copies of the variables.
        """
        import torch

        layers = list(layers)
        if not layers:
            raise ValueError("LinearGQ.fuse: no layers")
        first = layers[0]
        for layer in layers:
            if layer.variables is None:
                raise ValueError("LinearGQ.fuse: every layer needs its variables (build it or call init_variables)")
            if (layer.dim == 0) != (first.dim == 0):
                raise NotImplementedError("LinearGQ.fuse: layers grouped along different axes do not stack")
            if layer.group_size != first.group_size or layer.bias != first.bias:
                raise ValueError("LinearGQ.fuse: layers differ in group_size or bias")
            mine, theirs = layer.variables.weight_compressed.shape, first.variables.weight_compressed.shape
            if (mine[1:] != theirs[1:]) if first.dim == 0 else (mine[0] != theirs[0]):
                raise ValueError("LinearGQ.fuse: layers differ in input features")
        fused = cls(sum(l.out_features for l in layers), bias=first.bias, group_size=first.group_size, dim=first.dim)
        axis = 0 if first.dim == 0 else 1
        names = ["weight_compressed", "weight_decompression_scale", "weight_decompression_bias"]
        fused.variables = NamedTensors(
            **{n: Variable(n, torch.cat([l.variables[n].data for l in layers], dim=axis).contiguous()) for n in names}
        )
        if first.bias:
            fused.variables.insert("bias", Variable("bias", torch.cat([l.variables.bias.data for l in layers]).contiguous()))
        return fused

    @classmethod
    def fuse_inputs(cls, layers):
        """One layer computing the SUM of `layers`, each applied to its own slice of the input
        features: y = sum(l_i(x_i)) for x = cat([x_i], -1) (e.g. the attention output projection and
        the second feed-forward layer of a parallel decoder block, whose results are added: one
        product over [attention values ; feed-forward activations]).  The weights lie side by side
        along their input features: the variables stack along the group axis for dim=0 and along
        their first axis for dim=-1 / 1; the additive biases are summed in float32.  All layers
        must agree in dim, group_size, bias and output width.  The new layer owns its variables.
        """
        import torch

        layers = list(layers)
        if not layers:
            raise ValueError("LinearGQ.fuse_inputs: no layers")
        first = layers[0]
        for layer in layers:
            if layer.variables is None:
                raise ValueError("LinearGQ.fuse_inputs: every layer needs its variables (build it or call init_variables)")
            if (layer.dim == 0) != (first.dim == 0):
                raise NotImplementedError("LinearGQ.fuse_inputs: layers grouped along different axes do not stack")
            if layer.group_size != first.group_size or layer.bias != first.bias or layer.out_features != first.out_features:
                raise ValueError("LinearGQ.fuse_inputs: layers differ in group_size, bias or output features")
        fused = cls(first.out_features, bias=first.bias, group_size=first.group_size, dim=first.dim)
        axis = 1 if first.dim == 0 else 0
        names = ["weight_compressed", "weight_decompression_scale", "weight_decompression_bias"]
        fused.variables = NamedTensors(
            **{n: Variable(n, torch.cat([l.variables[n].data for l in layers], dim=axis).contiguous()) for n in names}
        )
        if first.bias:
            total = sum(l.variables.bias.data.float() for l in layers).to(first.variables.bias.data.dtype)
            fused.variables.insert("bias", Variable("bias", total.contiguous()))
        return fused

    def prepacked(self):
        """The weight in the streaming layout that `_gq_hip.GemvSequence.add` accepts in place of the
        three variables: a device copy of the same 0.5625 bytes per weight, made by
        gq_gemv_prepack_f16 (dim=0: group_size 64, input features a multiple of 512) or
        gq_gemv_kn_prepack_f16 (dim=-1 / 1, the default: group_size 64, input features a multiple of
        512; the output features are a multiple of 64 by construction).  The layer keeps its variables;
        make the copy again after `load_weights`."""
        if self.variables is None:
            raise ValueError("LinearGQ.prepacked: the layer has no variables yet (build it or call init_variables)")
        v = self.variables
        make = _gq_hip.prepack_gemv if self.dim == 0 else _gq_hip.prepack_gemv_kn
        return make(v.weight_compressed.data, v.weight_decompression_scale.data, v.weight_decompression_bias.data)

    def prepack_for_decode(self):
        """Keep a copy of the weight in the streaming layout of its dim (the price: a second copy of
        the packed weight); `load_weights` renews it.  Returns the copy (a `_gq_hip.PrepackedWeight`,
        which `GemvSequence.add` accepts).

        dim=-1 / 1 (the default layout): `build` then serves every batch from the copy
        (gq_linear_knp_act_f16: decode batches about twice as fast as the kernel that reads the
        variables, prefill batches through the MFMA pipeline of the other layout).
        dim=0: `build` hands the copy to gq_linear_p_act_f16 beside the variables; batches that run the
        pipelined GEMM kernel read it (5 - 12 % sooner, the same bits), single decode calls read the
        variables as before, and a `GemvSequence` streams the copy."""
        self._decode_copy = self.prepacked()
        return self._decode_copy

    # ------------------------------------------------------------------------- weight mapping

    @staticmethod
    def torch_mapping(variables: NamedTensors, nn_layer, dtype=None, group_size: int = 64, dim: int = -1) -> WeightsDict:
        """
        Mapping from the layer variables to the (compressed) torch.nn.Linear parameters
        (linear_gq.py:112-136).  `dtype` is the torch dtype of the additive bias (float32 if None).
        """
        import torch

        dtype = torch.float32 if dtype is None else dtype
        weight_t = nn_layer.weight.T.detach()
        if weight_t.is_cuda and weight_t.dtype in (torch.float16, torch.float32):
            # the packer on the device: the same bits as the numpy function gives for this array
            compressed = tuple(a.cpu().numpy() for a in group_quantize_compress(weight_t, group_size, dim=dim))
        else:
            # (any other dtype, e.g. float64: the numpy packer, as the reference does for every weight)
            compressed = group_quantize_compress_numpy(weight_t.cpu().numpy(), group_size, dim=dim)
        state_dict = dict(
            zip(
                (
                    variables.weight_compressed,
                    variables.weight_decompression_scale,
                    variables.weight_decompression_bias,
                ),
                compressed,
            )
        )
        if "bias" in variables.keys():
            state_dict[variables.bias] = nn_layer.bias.data.detach().cpu().numpy().astype(_numpy_dtype_of(dtype))
        return WeightsDict(state_dict)
