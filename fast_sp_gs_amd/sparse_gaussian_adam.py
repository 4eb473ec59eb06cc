"""SparseGaussianAdam: same class and behaviour as the reference's `fast_2d_gs/sparse_gaussian_adam.py` (lines 10-49),
driving the HIP masked-Adam kernel through the operator boundary."""
import torch
import torch.optim

from fast_sp_gs_amd._C import get_C_function

__all__ = ['SparseGaussianAdam']


class SparseGaussianAdam(torch.optim.Adam):
    _update_C = staticmethod(get_C_function('AdamMasksedUpdated'))

    def __init__(self, params, lr, eps):
        super().__init__(params=params, lr=lr, eps=eps)
        self.N = None
        self.visibility = None

    @torch.no_grad()
    def step(self):
        for group in self.param_groups:
            lr = group["lr"]
            eps = group["eps"]
            assert len(group["params"]) == 1, "more than one tensor in group"
            param = group["params"][0]
            if param.grad is None or param.grad.numel() == 0:
                continue
            state = self.state[param]
            if len(state) == 0:  # lazy state initialisation
                state['step'] = torch.tensor(0.0, dtype=torch.float32)
                state['exp_avg'] = torch.zeros_like(param, memory_format=torch.preserve_format)
                state['exp_avg_sq'] = torch.zeros_like(param, memory_format=torch.preserve_format)
            exp_avg, exp_avg_sq = state["exp_avg"], state["exp_avg_sq"]
            state['step'] += 1
            step = float(state['step'])
            M = param.numel() // self.N
            # bias corrections folded into the learning rate: lr * sqrt(1 - b2^t) / (1 - b1^t)
            self._update_C(param, param.grad, exp_avg, exp_avg_sq, self.visibility,
                           lr * (1 - 0.999 ** step) ** 0.5 / (1 - 0.9 ** step), 0.9, 0.999, eps, self.N, M)

    def set_before_step(self, visibility, N):
        self.visibility, self.N = visibility, N
