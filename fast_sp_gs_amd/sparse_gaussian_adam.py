"""SparseGaussianAdam: same class and behaviour as the reference's `fast_2d_gs/sparse_gaussian_adam.py` (lines 10-49),
driving the HIP masked-Adam kernel through the operator boundary."""
import numpy as np
import torch
import torch.optim

from fast_sp_gs_amd._C import get_C_function

__all__ = ['SparseGaussianAdam']


class SparseGaussianAdam(torch.optim.Adam):
    _update_C = staticmethod(get_C_function('AdamMasksedUpdated'))
    _update_multi_C = staticmethod(get_C_function('AdamMasksedUpdatedMulti'))
    _MAX = 12  # tensors per launch (fsgs_adam_masked_update_max_tensors)

    def __init__(self, params, lr, eps):
        super().__init__(params=params, lr=lr, eps=eps)
        self.N = None
        self.visibility = None

    def _advance(self, param):
        """The parameter's optimiser state with its step count advanced; created on first use with the keys torch's
        Adam uses (sparse_gaussian_adam.py:28-33), so checkpoints of either optimiser load into the other."""
        state = self.state[param]
        if not state:
            state.update(step=torch.zeros((), dtype=torch.float32),
                         exp_avg=torch.zeros_like(param, memory_format=torch.preserve_format),
                         exp_avg_sq=torch.zeros_like(param, memory_format=torch.preserve_format))
        state['step'] += 1
        return state

    @torch.no_grad()
    def step(self):
        """One masked Adam update of every parameter group that has a gradient (sparse_gaussian_adam.py:20-45), the
        groups' kernels folded into one launch per `_MAX` tensors; the arithmetic per element is the single-tensor
        kernel's."""
        jobs = []  # (param, grad, first moment, second moment, effective rate, eps)
        corrections = {}  # step count -> the two bias corrections, shared by the groups that are at that count
        for group in self.param_groups:
            if len(group["params"]) != 1:
                raise AssertionError("more than one tensor in group")
            param = group["params"][0]
            if param.grad is None or param.grad.numel() == 0:
                continue
            state = self._advance(param)
            # Bias corrections folded into the learning rate: lr * sqrt(1 - b2^t) / (1 - b1^t). The reference evaluates
            # this on the step count as a float32 tensor (sparse_gaussian_adam.py:42-46), so every operation rounds to
            # float32 and the product is widened to double at the call. The powers are taken by torch on the float32
            # tensor as there; the multiplication and division that follow are single correctly rounded float32
            # operations.
            t = state['step']
            key = float(t)
            if key not in corrections:
                corrections[key] = (np.float32(((1 - 0.999 ** t) ** 0.5).item()), np.float32((1 - 0.9 ** t).item()))
            root_c2, c1 = corrections[key]
            jobs.append((param, param.grad, state["exp_avg"], state["exp_avg_sq"],
                         float(np.float32(group["lr"]) * root_c2 / c1), group["eps"]))
        for i in range(0, len(jobs), self._MAX):
            p, g, m, v, rates, epss = map(list, zip(*jobs[i:i + self._MAX]))
            self._update_multi_C(p, g, m, v, self.visibility, rates, 0.9, 0.999, epss, self.N)

    def set_before_step(self, visibility, N):
        self.visibility, self.N = visibility, N
