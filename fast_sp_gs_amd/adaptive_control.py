"""Adaptive density control (densify / clone / split / prune) of a Gaussian point set on the compaction kernels.

Mirrors the methods of the reference's `GaussianSplatting` base model (fast_2d_gs/gaussian_splatting.py:486-642) and the
surfel-aware split of `network.py:1156-1193` -- same names, arguments, attribute names (`_xyz`, `_scaling`, ...,
`xyz_gradient_accum`, `denom`, `max_radii2D`, `param_names_map`) and the same resulting tensors, optimiser parameter
groups and Adam moments -- so a model class can take them over by inheriting from `AdaptiveControl`.

The reference performs every structural change tensor by tensor (`old[mask]`, `torch.cat`, `.repeat`) and moment by
moment: about 60 indexing launches for a prune, more for a densify. Here a change is one table `source_row[new_row]`
built from the masks (`select_indices`) and applied to all parameters, both Adam moments and the statistics by
`gather_rows` in one launch; `densify` merges the reference's clone -> split -> prune-the-split-parents sequence into a
single table (kept originals, clones, N blocks of children -- the order the sequence ends in).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch
from torch import Tensor, nn

from ._C import get_C_function


def inverse_sigmoid(x: Tensor) -> Tensor:
    return torch.log(x / (1 - x))


def _optimizers(optimizers) -> List[torch.optim.Optimizer]:
    return [optimizers] if isinstance(optimizers, torch.optim.Optimizer) else list(optimizers)


def restructure_optimizer(optimizers, names: Sequence[str], source_row: Tensor, new_rows: int = 0,
                          tail: Optional[Dict[str, Tensor]] = None) -> Dict[str, Tensor]:
    """Applies one row table to every named parameter group of the optimisers and to its Adam moments.

    New parameter = old[source_row]; the last `new_rows` rows are new points: their moments are zero (the reference
    concatenates `zeros_like`, gaussian_splatting.py:539-543); where `tail[name]` is given, the last `len(tail[name])`
    parameter rows are taken from it instead of from the table. Returns {group name: new nn.Parameter}, as `change_optimizer` does
    (gaussian_splatting.py:497-555).
    """
    gather = get_C_function('gather_rows')
    tail = tail or {}
    n_rows = source_row.shape[0]
    moment_row = source_row
    if new_rows:
        moment_row = source_row.clone()
        moment_row[n_rows - new_rows:] = -1
    groups, params, moments = [], [], []
    for optimizer in _optimizers(optimizers):
        for group in optimizer.param_groups:
            if group.get('name') not in names:
                continue
            old = group['params'][0]
            state = optimizer.state.get(old, None)
            groups.append((optimizer, group, old, state))
            params.append(old)
            if state is not None and 'exp_avg' in state:
                moments += [state['exp_avg'], state['exp_avg_sq']]
    if moment_row is source_row:  # no new rows: parameters and moments follow the same table, one launch
        both = gather(params + moments, source_row)
        new_params, new_moments = both[:len(params)], both[len(params):]
    else:
        new_params = gather(params, source_row)
        new_moments = gather(moments, moment_row) if moments else []
    out, k = {}, 0
    for (optimizer, group, old, state), new in zip(groups, new_params):
        name = group['name']
        if name in tail:
            new[n_rows - tail[name].shape[0]:] = tail[name]
        new = nn.Parameter(new.requires_grad_(True))
        group['params'][0] = new
        out[name] = new
        if state is None:
            continue
        del optimizer.state[old]
        if 'exp_avg' in state:
            state['exp_avg'], state['exp_avg_sq'] = new_moments[k], new_moments[k + 1]
            k += 2
        optimizer.state[new] = state
    return out


class AdaptiveControl:
    """Mixin with the reference's density-control methods. The host class provides the six parameters named in
    `param_names_map`, the buffers `xyz_gradient_accum` [P,1], `denom` [P,1], `max_radii2D` [P] and the activations
    `get_scaling` / `get_opacity`; `is_surfel` says whether a split treats the third axis as flat (network.py:1170-1172).
    """
    param_names_map = {'_xyz': 'xyz', '_features_dc': 'f_dc', '_features_rest': 'f_rest', '_scaling': 'scaling',
                       '_rotation': 'rotation', '_opacity': 'opacity'}
    is_surfel = True
    # Per-point tensors of the host class that are not optimised but have to follow every structural change: a new point
    # takes its parent's row, a pruned point's row goes. The superpoint model keeps three of them -- the per-frame culling
    # flags, the visibility factor of the gradient statistics and the superpoint assignment (network.py:1195-1215) --
    # which the reference carries along with `t[valid]` / `cat((t, t[mask]))` / `cat((t, t[mask].repeat(N, 1)))`. Here they
    # go through the same row table as the parameters; attributes that are absent, None or empty are skipped.
    per_point_buffers = ('_culling', 'factor_culling', 'p2sp')

    @property
    def get_scaling(self) -> Tensor:
        return torch.exp(self._scaling)

    @property
    def get_opacity(self) -> Tensor:
        return torch.sigmoid(self._opacity)

    @property
    def points(self) -> Tensor:
        return self._xyz

    # ---- statistics ------------------------------------------------------------------------------------------------
    def training_setup(self):
        """gaussian_splatting.py:478-484."""
        P, dev = self._xyz.shape[0], self._xyz.device
        self.max_radii2D = torch.zeros((P,), device=dev)
        self.xyz_gradient_accum = torch.zeros((P, 1), device=dev)
        self.denom = torch.zeros((P, 1), device=dev)

    @torch.no_grad()
    def update_statistics(self, radii: Tensor, viewspace_grad: Tensor, factor: Optional[Tensor] = None) -> Tensor:
        """The per-step part of `adaptive_control` (network.py:1276-1282, gaussian_splatting.py:486-495) in one launch;
        returns the visibility mask `radii > 0` that the optimiser's `set_before_step` takes."""
        if radii.ndim == 2:
            radii = radii.amax(dim=0)
        return get_C_function('densification_stats')(radii.contiguous(), viewspace_grad.contiguous(), self.max_radii2D,
                                                     self.xyz_gradient_accum, self.denom, factor)

    def add_densification_stats(self, viewspace_point_tensor, update_filter: Tensor):
        """gaussian_splatting.py:486-495, signature kept; `update_filter` is a bool mask."""
        if isinstance(viewspace_point_tensor, Tensor):
            grad = viewspace_point_tensor.grad
        elif len(viewspace_point_tensor) == 1:
            grad = viewspace_point_tensor[0].grad
        else:
            grad = torch.zeros_like(viewspace_point_tensor[0])
            for p in viewspace_point_tensor:
                grad += p.grad
        # the kernel reads "radii > 0": hand it the filter as 0 / 1 radii and leave max_radii2D alone
        scratch = torch.zeros_like(self.max_radii2D)
        # the superpoint model weighs a point's gradient norm by its visibility factor (network.py:1153)
        factor = getattr(self, 'factor_culling', None)
        if factor is not None and factor.numel() != self._xyz.shape[0]:
            factor = None
        get_C_function('densification_stats')(update_filter.to(torch.int32), grad.contiguous(), scratch,
                                              self.xyz_gradient_accum, self.denom,
                                              None if factor is None else factor.reshape(-1).contiguous())

    # ---- structural changes ------------------------------------------------------------------------------------------
    def _restructure(self, optimizer, source_row: Tensor, new_rows: int = 0, tail: Optional[Dict[str, Tensor]] = None,
               reset_statistics: bool = False):
        P_old = self._xyz.shape[0]
        new = restructure_optimizer(optimizer, list(self.param_names_map.values()), source_row, new_rows, tail)
        for param_name, opt_name in self.param_names_map.items():
            setattr(self, param_name, new[opt_name])
        carried = [n for n in self.per_point_buffers
                   if isinstance(getattr(self, n, None), Tensor) and getattr(self, n).ndim >= 1 and
                   getattr(self, n).shape[0] == P_old and P_old > 0]
        if carried:
            # densification_postfix marks its appended rows -1 (they come from `tail`); such rows have no parent to copy
            # from, so they read zeros, as a model that appends foreign points has to fill them itself anyway
            for n, t in zip(carried, get_C_function('gather_rows')([getattr(self, n) for n in carried], source_row)):
                setattr(self, n, t)
        if reset_statistics:  # gaussian_splatting.py:575-578
            self.training_setup()
        else:  # gaussian_splatting.py:566-568
            self.xyz_gradient_accum, self.denom, self.max_radii2D = get_C_function('gather_rows')(
                [self.xyz_gradient_accum, self.denom, self.max_radii2D], source_row)

    def prune_points(self, optimizer, mask: Tensor):
        """gaussian_splatting.py:557-568: drops the points whose mask entry is set."""
        self._restructure(optimizer, get_C_function('select_indices')(mask, True))

    def densification_postfix(self, optimizer, mask=None, N=None, **kwargs):
        """gaussian_splatting.py:570-579: appends the given rows (keyed by optimiser group name)."""
        P = self._xyz.shape[0]
        n_new = next(iter(kwargs.values())).shape[0]
        rows = torch.arange(P + n_new, dtype=torch.int32, device=self._xyz.device)
        rows[P:] = -1
        self._restructure(optimizer, rows, n_new, kwargs, reset_statistics=True)
        return mask

    def _children(self, selected: Tensor, N: int, noise: Optional[Tensor]):
        scaling = self.get_scaling
        if not self.is_surfel and scaling.shape[1] != 3:
            raise RuntimeError('a 3D Gaussian needs three scales')
        if noise is None:  # the draws of torch.normal(mean=0, std=stds), gaussian_splatting.py:592
            noise = torch.randn((selected.numel() * N, 3), device=self._xyz.device)
        return get_C_function('split_children')(selected, N, self._xyz.detach(), scaling.detach().contiguous(),
                                                self._rotation.detach(), noise)

    def densify_and_clone(self, optimizer, grads, grad_threshold, scene_extent):
        """gaussian_splatting.py:610-621."""
        selected_pts_mask = (torch.norm(grads, dim=-1) >= grad_threshold) & \
                            (torch.amax(self.get_scaling, dim=1) <= scene_extent)
        P = self._xyz.shape[0]
        sel = get_C_function('select_indices')(selected_pts_mask)
        rows = torch.cat([torch.arange(P, dtype=torch.int32, device=sel.device), sel])
        self._restructure(optimizer, rows, sel.numel(), reset_statistics=True)
        return selected_pts_mask

    def densify_and_split(self, optimizer, grads, grad_threshold, scene_extent, N=2, noise: Optional[Tensor] = None):
        """gaussian_splatting.py:581-608 / network.py:1156-1193: N children per selected point, parents removed."""
        P, dev = self._xyz.shape[0], self._xyz.device
        padded_grad = torch.zeros((P,), device=dev)
        padded_grad[:grads.shape[0]] = grads.squeeze(-1) if grads.ndim > 1 else grads
        selected_pts_mask = (padded_grad >= grad_threshold) & (torch.amax(self.get_scaling, dim=1) > scene_extent)
        select = get_C_function('select_indices')
        sel, keep = select(selected_pts_mask), select(selected_pts_mask, True)
        new_xyz, new_scaling = self._children(sel, N, noise)
        rows = torch.cat([keep, sel.repeat(N)])
        self._restructure(optimizer, rows, sel.numel() * N,
                    {self.param_names_map['_xyz']: new_xyz, self.param_names_map['_scaling']: new_scaling},
                    reset_statistics=True)

    def densify(self, optimizer, max_grad: float, extent: float, densify_percent_dense=0.01, N: int = 2,
                noise: Optional[Tensor] = None):
        """gaussian_splatting.py:623-628: clone, then split, as one restructuring. Clones enter the split test with a zero
        gradient (the reference pads, :585-586), so for a positive threshold they are never split and the final order is
        kept originals, clones, children; a non-positive threshold takes the two-step route."""
        scale_threshold = densify_percent_dense * extent
        if not max_grad > 0:
            grads = self.xyz_gradient_accum / self.denom
            grads[grads.isnan()] = 0.0
            self.densify_and_clone(optimizer, grads, max_grad, scale_threshold)
            self.densify_and_split(optimizer, grads, max_grad, scale_threshold, N, noise)
            return
        clone_mask, split_mask = get_C_function('densify_masks')(
            self.xyz_gradient_accum, self.denom, self.get_scaling.detach().contiguous(), max_grad, scale_threshold)
        select = get_C_function('select_indices')
        clones, parents, keep = select(clone_mask), select(split_mask), select(split_mask, True)
        new_xyz, new_scaling = self._children(parents, N, noise)
        n_children = parents.numel() * N
        rows = torch.cat([keep, clones, parents.repeat(N)])
        self._restructure(optimizer, rows, clones.numel() + n_children,
                    {self.param_names_map['_xyz']: new_xyz, self.param_names_map['_scaling']: new_scaling},
                    reset_statistics=True)

    def prune(self, optimizer, min_opacity: float, extent: float, max_screen_size, prune_percent_dense=0.1):
        """gaussian_splatting.py:630-636."""
        mask = get_C_function('prune_mask')(self.get_opacity.detach().contiguous(), self.max_radii2D,
                                            self.get_scaling.detach().contiguous(), min_opacity, max_screen_size,
                                            prune_percent_dense * extent)
        self.prune_points(optimizer, mask)

    def reset_opacity(self, optimizer):
        """gaussian_splatting.py:638-641: opacities capped at 0.01, their Adam moments cleared."""
        opacities_new = inverse_sigmoid(torch.min(self.get_opacity, torch.ones_like(self.get_opacity) * 0.01)).detach()
        name = self.param_names_map['_opacity']
        for opt in _optimizers(optimizer):
            for group in opt.param_groups:
                if group.get('name') != name:
                    continue
                old = group['params'][0]
                new = nn.Parameter(opacities_new.requires_grad_(True))
                group['params'][0] = new
                state = opt.state.get(old, None)
                if state is not None:
                    del opt.state[old]
                    if 'exp_avg' in state:
                        state['exp_avg'] = torch.zeros_like(new)
                        state['exp_avg_sq'] = torch.zeros_like(new)
                    opt.state[new] = state
                self._opacity = new


class GaussianPoints(nn.Module, AdaptiveControl):
    """Minimal holder of the six per-point parameters with the reference's names (gaussian_splatting.py:78-140)."""

    def __init__(self, xyz: Tensor, features_dc: Tensor, features_rest: Tensor, scaling: Tensor, rotation: Tensor,
                 opacity: Tensor, is_surfel: Optional[bool] = None):
        super().__init__()
        self._xyz = nn.Parameter(xyz.clone())
        self._features_dc = nn.Parameter(features_dc.clone())
        self._features_rest = nn.Parameter(features_rest.clone())
        self._scaling = nn.Parameter(scaling.clone())
        self._rotation = nn.Parameter(rotation.clone())
        self._opacity = nn.Parameter(opacity.clone())
        self.is_surfel = scaling.shape[1] == 2 if is_surfel is None else is_surfel
        self.training_setup()

    def param_groups(self, lr: float = 1e-3):
        return [{'params': [getattr(self, a)], 'lr': lr, 'name': n} for a, n in self.param_names_map.items()]
