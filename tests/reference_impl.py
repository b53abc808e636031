"""Oracle-backed reference implementations for the benchmark harness (tests only): objects with
the numpy entry points the harness calls on its ``reference_implementation`` (the role e3nn plays
in the reference: implementations/E3NNTensorProduct.py, convolution/E3NNConv.py)."""
import numpy as np

from oracle import spec, tp as otp


def _oracle_problem(config):
    # the instructions as the user gave them: after construction the product's own list carries
    # the normalisation coefficients in place of the user's path weights
    ins = [tuple(t)[:6] for t in config.instructions_raw]
    return spec.Problem(str(config.irreps_in1), str(config.irreps_in2), str(config.irreps_out), ins,
                        in1_var=config.in1_var, in2_var=config.in2_var, out_var=config.out_var,
                        irrep_normalization=config.irrep_normalization, path_normalization=config.path_normalization,
                        shared_weights=bool(config.shared_weights))


class OracleTensorProduct:
    def __init__(self, config, torch_op=False):
        self.config, self.oprob = config, _oracle_problem(config)

    @staticmethod
    def name():
        return "Oracle"

    def forward_cpu(self, L1_in, L2_in, L3_out, weights):
        L3_out[...] = otp.forward(self.oprob, L1_in, L2_in, weights)

    def backward_cpu(self, L1_in, L1_grad, L2_in, L2_grad, L3_grad, weights, weights_grad):
        dX, dY, dW = otp.backward(self.oprob, L1_in, L2_in, weights, L3_grad)
        L1_grad[...], L2_grad[...], weights_grad[...] = dX, dY, dW


class OracleConv:
    deterministic = False

    def __init__(self, config, torch_op=False):
        self.config, self.oprob = config, _oracle_problem(config)

    @staticmethod
    def name():
        return "OracleConv"

    def forward_cpu(self, L1_in, L2_in, weights, L3_out, graph):
        L3_out[...] = otp.conv_forward(self.oprob, L1_in, L2_in, weights, graph.rows, graph.cols)

    def backward_cpu(self, L1_in, L1_grad, L2_in, L2_grad, L3_grad, weights, weights_grad, graph):
        dX, dY, dW = otp.conv_backward(self.oprob, L1_in, L2_in, weights, L3_grad, graph.rows, graph.cols)
        L1_grad[...], L2_grad[...], weights_grad[...] = dX, dY, dW


class TorchReferenceTP(OracleTensorProduct):
    """Differentiable fp64 CPU reference for the second-order checks."""
    device = "cpu"

    def __init__(self, config, torch_op=True):
        import torch
        from oracle.torch_cpu import TorchTP
        super().__init__(config)
        self._tp = TorchTP(self.oprob, dtype=torch.float64)

    def forward(self, L1_in, L2_in, weights):
        return self._tp.forward(L1_in.double(), L2_in.double(), weights.double()).to(L1_in.dtype)


class TorchReferenceConv(OracleConv):
    device = "cpu"

    def __init__(self, config, torch_op=True):
        import torch
        from oracle.torch_cpu import TorchTP
        super().__init__(config)
        self._tp = TorchTP(self.oprob, dtype=torch.float64)

    def forward(self, L1_in, L2_in, weights, rows, cols):
        return self._tp.conv_forward(L1_in.double(), L2_in.double(), weights.double(), rows, cols).to(L1_in.dtype)
