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

    @torch.no_grad()
    def step(self):
        """The reference's loop over parameter groups (sparse_gaussian_adam.py:20-45), with the groups' kernels folded
        into one launch per `_MAX` tensors; the arithmetic per element is the single-tensor kernel's."""
        params, grads, ms, vs, lrs, epss = [], [], [], [], [], []
        corrections = {}  # step count -> the two bias corrections, shared by the groups that are at that count
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
            state['step'] += 1
            step = state['step']
            params.append(param), grads.append(param.grad), ms.append(state["exp_avg"]), vs.append(state["exp_avg_sq"])
            # Bias corrections folded into the learning rate: lr * sqrt(1 - b2^t) / (1 - b1^t). The reference evaluates
            # this on `step`, a float32 tensor (sparse_gaussian_adam.py:42-46), so every operation rounds to float32
            # and the product is widened to double at the call. The powers are taken by torch on the float32 tensor as
            # there; the multiplication and division that follow are single correctly rounded float32 operations.
            key = float(step)
            if key not in corrections:
                corrections[key] = (np.float32(((1 - 0.999 ** step) ** 0.5).item()),
                                    np.float32((1 - 0.9 ** step).item()))
            root_c2, c1 = corrections[key]
            lrs.append(float(np.float32(lr) * root_c2 / c1))
            epss.append(eps)
        for i in range(0, len(params), self._MAX):
            j = slice(i, i + self._MAX)
            self._update_multi_C(params[j], grads[j], ms[j], vs[j], self.visibility, lrs[j], 0.9, 0.999, epss[j], self.N)

    def set_before_step(self, visibility, N):
        self.visibility, self.N = visibility, N
