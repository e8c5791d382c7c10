"""Batch inference from a model directory, the reference's `staf_full_inference` on top of the PyTorch layer shells.

Mirrors STAF/staf_models/staf_model_inference_full.py:36-182 (constructor from the model directory, `full_test`,
`energy_of_n_atoms`) and the exported per-species network wrapper `TestModel.testmodel`
(STAF/save_models/save_model_in_double.py:22-36).  The reference loads each species' network as a TF SavedModel
(`model_type{k}`); here the Dense stack comes from `mlp_type{k}.bin` of the same directory, the file its MD library
reads.  Everything runs on the GPU: descriptor op, fingerprints, network (torch), force and virial ops.
"""
import os

import numpy as np
import torch

from . import model_dir
from .layers import descriptor_layer, force_virial_layer, physics_layer


def make_typemap(tipos):
    """Species index of every atom of a species-sorted frame (staf_model_inference_full.py:23-33)."""
    tipos = np.atleast_1d(np.asarray(tipos, dtype=np.int64))
    return np.concatenate([np.full(int(n), k, dtype=np.int32) for k, n in enumerate(tipos)])


class TestModel(torch.nn.Module):
    """log(AF + 1e-3) - mu -> Dense stack; `testmodel` returns (1/2 sum of the atomic energies [B], d(sum e)/dAF)."""
    __test__ = False   # not a pytest class

    def __init__(self, mu, layers, dtype, device):
        super().__init__()
        T = lambda a: torch.nn.Parameter(torch.as_tensor(np.asarray(a), dtype=dtype, device=device),
                                         requires_grad=False)
        self.alphamu = T(mu)
        self.W = torch.nn.ParameterList([T(W) for W, _, _ in layers])
        self.b = torch.nn.ParameterList([T(b) for _, b, _ in layers])
        self.act = [a for _, _, a in layers]

    def testmodel(self, des):
        with torch.enable_grad():
            des = des.detach().requires_grad_(True)
            x = torch.log(des + 1e-3) - self.alphamu
            for W, b, act in zip(self.W, self.b, self.act):
                x = x @ W + b
                if act == "tanh":
                    x = torch.tanh(x)
                elif act == "relu":
                    x = torch.relu(x)
            energies = x[..., 0]
            grad, = torch.autograd.grad(energies.sum(), des)
        return 0.5 * energies.detach().sum(dim=1), grad


class staf_full_inference(torch.nn.Module):
    """Energy, forces and the full virial tensor of batches of species-sorted frames."""

    def __init__(self, modelname, max_batch=1, dtype=torch.float64, device="cuda:0"):
        super().__init__()
        self.dtype, self.device = dtype, torch.device(device)
        self.max_batch = max_batch
        tip = np.loadtxt(os.path.join(modelname, "type.dat"), dtype=np.int64).reshape(-1)
        self.ntipos = len(tip)
        self.nt_couple = self.ntipos * (self.ntipos + 1) // 2
        ci = np.loadtxt(os.path.join(modelname, "cutoff_info"))
        self.rc, self.rad_buff = float(ci[0, 0]), int(ci[0, 1])
        self.rc_ang, self.ang_buff = float(ci[1, 0]), int(ci[1, 1])
        self.rs = float(ci[2, 0])
        self.tipos = torch.as_tensor(tip, dtype=torch.int32, device=self.device)
        self._counts = [int(n) for n in tip]
        self.type_map = torch.as_tensor(make_typemap(tip), device=self.device)
        self.N = int(self.type_map.shape[0])
        self.boxinit = torch.tensor([12., 0., 0., 12., 0., 12.], dtype=dtype, device=self.device)
        self.descriptor_layer = descriptor_layer(self.rc, self.rad_buff, self.rc_ang, self.ang_buff, self.N,
                                                 self.boxinit, self.rs, self.max_batch, dtype=dtype)
        _, species = model_dir.read_model_dir(modelname)
        T = lambda a: torch.as_tensor(np.asarray(a), dtype=dtype, device=self.device)
        # the layers square their embeddings; the directory's squared files are what the kernels must see
        self.physics_layer = torch.nn.ModuleList(
            [physics_layer(T(sp["alpha2b"]), T(sp["alpha3b"]), [T(np.sqrt(sp["emb2b"])), T(np.sqrt(sp["emb3b"]))])
             for sp in species])
        self.nets = torch.nn.ModuleList([TestModel(sp["mu"], sp["layers"], dtype, self.device) for sp in species])
        self.force_layer = force_virial_layer(self.rad_buff, self.ang_buff, with_grad=False)

    @torch.no_grad()
    def full_test(self, pos, box, energy_only=False):
        """pos [B, 3N], box [B, 6] -> (energy [B], force [B, 3N], virial [B, 9] row-major); energy_only: forces and
        virial are zeros."""
        pos = torch.as_tensor(pos, dtype=self.dtype, device=self.device)
        box = torch.as_tensor(box, dtype=self.dtype, device=self.device)
        x1, x2, x3bsupp, int2b, int3b, intder2b, intder3b, intder3bsupp, numtriplet = self.descriptor_layer(pos, box)
        B = pos.shape[0]
        energy = torch.zeros(B, dtype=self.dtype, device=self.device)
        force = torch.zeros((B, 3 * self.N), dtype=self.dtype, device=self.device)
        virial = torch.zeros((B, 9), dtype=self.dtype, device=self.device)
        o = 0
        for k in range(self.ntipos):
            s = slice(o, o + self._counts[k])
            o = s.stop
            pl = self.physics_layer[k]
            fingers = pl(x1[:, s], x3bsupp[:, s], int2b[:, s], x2[:, s], int3b[:, s], numtriplet[:, s],
                         self.type_map)
            e, g = self.nets[k].testmodel(fingers)
            energy += e
            if energy_only:
                continue
            f, w = self.force_layer(g[..., :pl.nalpha_r].contiguous(), x1[:, s], intder2b[:, s], int2b[:, s],
                                    pl.alpha2b, g[..., pl.nalpha_r:].contiguous(), x2[:, s], x3bsupp[:, s],
                                    intder3b[:, s], intder3bsupp[:, s], int3b[:, s], numtriplet[:, s], pl.alpha3b,
                                    pl.type_emb_2b, pl.type_emb_3b, self.type_map, self.tipos, k, pos, box)
            force += f
            virial += w
        return energy, force, virial

    @torch.no_grad()
    def energy_of_n_atoms(self, pos_n, types_n, box6):
        """Energy of an n-atom configuration given in any atom order (staf_model_inference_full.py:146-182)."""
        pos_n = np.asarray(pos_n, dtype=np.float64).reshape(-1, 3)
        types_n = np.asarray(types_n, dtype=np.int32).reshape(-1)
        if pos_n.shape[0] < 1:
            return 0.0
        order = np.argsort(types_n, kind="stable")
        counts = np.bincount(types_n[order], minlength=self.ntipos)
        type_map = torch.as_tensor(types_n[order], device=self.device)
        pos = torch.as_tensor(pos_n[order].reshape(1, -1), dtype=self.dtype, device=self.device)
        box = torch.as_tensor(np.asarray(box6, dtype=np.float64).reshape(1, 6), dtype=self.dtype, device=self.device)
        x1, x2, x3bsupp, int2b, int3b, _d2, _d3, _d3s, numtriplet = self.descriptor_layer(pos, box)
        tot, start = 0.0, 0
        for k in range(self.ntipos):
            nk = int(counts[k])
            if nk == 0:
                continue
            s = slice(start, start + nk)
            start += nk
            fingers = self.physics_layer[k](x1[:, s], x3bsupp[:, s], int2b[:, s], x2[:, s], int3b[:, s],
                                            numtriplet[:, s], type_map)
            tot += float(self.nets[k].testmodel(fingers)[0][0])
        return tot
