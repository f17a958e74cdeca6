"""nn.MLP and the functional mlp(): the host-side mirror of endia/nn/modules/_mlp.mojo."""
from . import functional as F


class MLP:
    """Dense stack `pred = act(pred @ W_i + b_i)` with no activation after the last layer
    (_mlp.mojo:47-53). W_i is [in, out], b_i is [out]; BOTH are He-normal with std sqrt(2 / fan_in)
    (_mlp.mojo:30-43). The reference hard-codes ReLU; `activation` also accepts "tanh", "sin" and None.

    `fused=True` (default) evaluates each layer as one GEMM with a bias + activation epilogue;
    `fused=False` issues the reference's op sequence matmul -> add -> activation;
    `fused="model"` evaluates the WHOLE stack as one op (functional.mlp_forward): for small models (widths up to 128,
    relu / tanh / no activation) that is one launch forward and two backward; first-order passes only.
    """

    def __init__(self, hidden_dims, compute_backward=False, activation="relu", fused=True):
        self.hidden_dims = list(hidden_dims)
        self.num_layers = len(hidden_dims) - 1
        self.compute_backward = compute_backward
        self.activation = activation
        self.fused = fused
        self.weights, self.biases = [], []
        for i in range(self.num_layers):
            self.weights.append(F.rand_he_normal([hidden_dims[i], hidden_dims[i + 1]], fan_in=hidden_dims[i],
                                                 requires_grad=compute_backward))
            self.biases.append(F.rand_he_normal([hidden_dims[i + 1]], fan_in=hidden_dims[i],
                                                requires_grad=compute_backward))

    def forward(self, x):
        if self.fused == "model":
            return F.mlp_forward(x, self.weights, self.biases, self.activation)
        pred = x
        act_fn = {"relu": F.relu, "tanh": F.tanh, "sin": F.sin, None: None}[self.activation]
        for i in range(self.num_layers):
            last = i == self.num_layers - 1
            if self.fused:
                pred = F.linear(pred, self.weights[i], self.biases[i], None if last else self.activation)
            else:
                pred = pred @ self.weights[i] + self.biases[i]
                if not last and act_fn is not None:
                    pred = act_fn(pred)
        return pred

    __call__ = forward

    def mse_loss(self, x, target):
        """mse(self.forward(x), target). With fused="model" and a small model the forward launch evaluates the loss
        and its gradient as well (functional.mlp_mse_loss): a training step is then forward + loss, cotangents,
        gradients and the optimizer, four launches."""
        if self.fused == "model":
            return F.mlp_mse_loss(x, target, self.weights, self.biases, self.activation)
        return F.mse(self.forward(x), target)

    def params(self):
        out = []
        for w, b in zip(self.weights, self.biases):
            out += [w, b]
        return out


def mlp(args):
    """Functional form (_mlp.mojo:71-82): args = [x, target, W_0, b_0, W_1, b_1, ...]."""
    pred = args[0]
    n = (len(args) - 2) // 2
    for i in range(n):
        pred = pred @ args[2 + 2 * i] + args[3 + 2 * i]
        if i < n - 1:
            pred = F.relu(pred)
    return pred
