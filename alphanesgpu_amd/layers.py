"""PyTorch shells of the reference's Python layers, with its gradient routing.

The reference wires its ops into TensorFlow through `tf.Module` layers (STAF/source_routine/descriptor_builder.py,
physics_layer_mod.py, force_layer_mod.py) and `RegisterGradient` entries (STAF/gradient_utility/*.py).  The classes
here have the same names, constructor arguments and call signatures on top of `alphanesgpu_amd.ops`, as
`torch.nn.Module`s, and the same routing as `torch.autograd.Function`s:

    op                       gradient op                       gradients returned for
    ComputeSortProj          ComputeTwoBodyParGrad             alpha2b, emb2b             register_2bAFs_grad.py:14-21
    ComputeSortProj3body     ComputeSortProj3bodyGrad          alpha3b, emb3b             register_3bAFs_grad.py:14-22
    ComputeForceRadial       ComputeForceRadialGrad            netderiv, alpha2b, emb2b   register_force_2bAFs_grad.py:14-24
    ComputeForceTripl        ComputeForceTriplGrad             netderiv, alpha3b, emb3b   register_force_3bAFs_grad.py:14-24
    ...Virial forms          ...VirialGrad                     the same                   register_force_*_virial_grad.py

`descriptor_physics_layer` runs the descriptor op and the two fingerprint ops of all species as one launch and routes
the same gradient ops.  Descriptors, maps and positions receive no gradient (the reference returns None for them): the descriptor op is not
differentiated, forces come from the stored Jacobians.  Every tensor lives on the GPU; the ops run on torch's current
stream.
"""
import torch

from . import ops


class _SortProj(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x2b, intmap2b, alpha2b, emb2b_sq, type_map):
        ctx.save_for_backward(x2b, intmap2b, alpha2b, emb2b_sq, type_map)
        return ops.compute_sort_proj(x2b, intmap2b, alpha2b, emb2b_sq, type_map)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad):
        x2b, intmap2b, alpha2b, emb2b_sq, type_map = ctx.saved_tensors
        ga, ge = ops.compute_two_body_par_grad(grad.contiguous(), x2b, intmap2b, alpha2b, emb2b_sq, type_map)
        return None, None, ga, ge, None


class _SortProj3body(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x3b, x3bsupp, intmap3b, intmap2b, alpha3b, emb3b_sq, type_map, numtriplet):
        ctx.save_for_backward(x3b, x3bsupp, intmap3b, intmap2b, alpha3b, emb3b_sq, type_map, numtriplet)
        ctx.nt = ops._nt_from_ntc(alpha3b.shape[0])
        return ops.compute_sort_proj3body(x3b, x3bsupp, intmap3b, intmap2b, alpha3b, emb3b_sq, type_map, numtriplet,
                                          nt=ctx.nt)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad):
        x3b, x3bsupp, intmap3b, intmap2b, alpha3b, emb3b_sq, type_map, numtriplet = ctx.saved_tensors
        ga, ge = ops.compute_sort_proj3body_grad(grad.contiguous(), x3b, x3bsupp, intmap3b, intmap2b, alpha3b,
                                                 emb3b_sq, type_map, numtriplet, nt=ctx.nt)
        return None, None, None, None, ga, ge, None, None


class _ForceRadial(torch.autograd.Function):
    """ComputeForceRadial, or ComputeForceRadialVirial when pos and box are given (two outputs then)."""

    @staticmethod
    def forward(ctx, netderiv, intder2b, intmap2b, x2b, alpha2b, emb2b_sq, type_map, tipos, type_now, pos, box):
        ctx.save_for_backward(netderiv, intder2b, intmap2b, x2b, alpha2b, emb2b_sq, type_map, tipos, type_now, pos,
                              box)
        out = ops.compute_force_radial(netderiv, intder2b, intmap2b, x2b, alpha2b, emb2b_sq, type_map, tipos,
                                       type_now, pos, box)
        if pos is None:
            return out
        ctx.shapes = (out[0].shape, out[1].shape)
        return out

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_force, grad_virial=None):
        netderiv, intder2b, intmap2b, x2b, alpha2b, emb2b_sq, type_map, tipos, type_now, pos, box = ctx.saved_tensors
        if pos is None:
            gn, ga, ge = ops.compute_force_radial_grad(grad_force.contiguous(), netderiv, intder2b, intmap2b, x2b,
                                                       alpha2b, emb2b_sq, type_map, tipos, type_now)
        else:
            # a missing branch counts as zero (register_force_2bAFs_virial_grad.py:15-18)
            gf = grad_force if grad_force is not None else x2b.new_zeros(ctx.shapes[0])
            gv = grad_virial if grad_virial is not None else x2b.new_zeros(ctx.shapes[1])
            gn, ga, ge = ops.compute_force_radial_virial_grad(gf.contiguous(), gv.contiguous(), netderiv, intder2b,
                                                              intmap2b, x2b, alpha2b, emb2b_sq, type_map, tipos,
                                                              type_now, pos, box)
        return gn, None, None, None, ga, ge, None, None, None, None, None


class _ForceTripl(torch.autograd.Function):
    """ComputeForceTripl, or ComputeForceTriplVirial when pos and box are given (two outputs then)."""

    @staticmethod
    def forward(ctx, netderiv, x3bsupp, x3b, intder3bsupp, intder3b, intmap2b, intmap3b, alpha3b, emb3b_sq, type_map,
                tipos, type_now, numtriplet, pos, box):
        ctx.save_for_backward(netderiv, x3bsupp, x3b, intder3bsupp, intder3b, intmap2b, intmap3b, alpha3b, emb3b_sq,
                              type_map, tipos, type_now, numtriplet, pos, box)
        out = ops.compute_force_tripl(netderiv, x3bsupp, x3b, intder3bsupp, intder3b, intmap2b, intmap3b, alpha3b,
                                      emb3b_sq, type_map, tipos, type_now, numtriplet, pos, box)
        if pos is None:
            return out
        ctx.shapes = (out[0].shape, out[1].shape)
        return out

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_force, grad_virial=None):
        (netderiv, x3bsupp, x3b, intder3bsupp, intder3b, intmap2b, intmap3b, alpha3b, emb3b_sq, type_map, tipos,
         type_now, numtriplet, pos, box) = ctx.saved_tensors
        if pos is None:
            gn, ga, ge = ops.compute_force_tripl_grad(grad_force.contiguous(), netderiv, x3bsupp, x3b, intder3bsupp,
                                                      intder3b, intmap2b, intmap3b, alpha3b, emb3b_sq, type_map,
                                                      tipos, type_now, numtriplet)
        else:
            gf = grad_force if grad_force is not None else x3b.new_zeros(ctx.shapes[0])
            gv = grad_virial if grad_virial is not None else x3b.new_zeros(ctx.shapes[1])
            gn, ga, ge = ops.compute_force_tripl_virial_grad(gf.contiguous(), gv.contiguous(), netderiv, x3bsupp, x3b,
                                                             intder3bsupp, intder3b, intmap2b, intmap3b, alpha3b,
                                                             emb3b_sq, type_map, tipos, type_now, numtriplet, pos,
                                                             box)
        return gn, None, None, None, None, None, None, ga, ge, None, None, None, None, None, None


class _DescriptorsFingerprints(torch.autograd.Function):
    """ComputeDescriptorsLight, then ComputeSortProj3body and ComputeSortProj for every centre species, as one launch
    (ops.compute_descriptors_fingerprints).  Outputs: the nine descriptor tensors (no gradient), then per species
    the 3-body fingerprints, then per species the 2-body fingerprints; gradients go to the parameter tensors through
    the gradient ops of the two fingerprint ops, species by species, exactly as from _SortProj3body / _SortProj."""

    @staticmethod
    def forward(ctx, pos, box, type_map, n_local, *params):
        nt = len(n_local)
        a3, e3, a2, e2 = (list(params[i * nt:(i + 1) * nt]) for i in range(4))
        desc, af3, af2 = ops.compute_descriptors_fingerprints(pos, box, type_map, n_local, a3, e3, a2, e2)
        ctx.n_local = [int(n) for n in n_local]
        ctx.save_for_backward(type_map, *desc, *params)
        ctx.mark_non_differentiable(*desc)
        return (*desc, *af3, *af2)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, *grads):
        nt = len(ctx.n_local)
        type_map = ctx.saved_tensors[0]
        rad, ang, sup, im2, im3, _, _, _, ntr = ctx.saved_tensors[1:10]
        params = ctx.saved_tensors[10:]
        a3, e3, a2, e2 = (params[i * nt:(i + 1) * nt] for i in range(4))
        g3, g2 = grads[9:9 + nt], grads[9 + nt:9 + 2 * nt]
        ga3, ge3, ga2, ge2 = [], [], [], []
        first = 0
        for k, n in enumerate(ctx.n_local):
            s = slice(first, first + n)
            first += n
            if g3[k] is None or n == 0:
                ga3.append(None), ge3.append(None)
            else:
                a, e = ops.compute_sort_proj3body_grad(g3[k].contiguous(), ang[:, s], sup[:, s], im3[:, s], im2[:, s],
                                                       a3[k], e3[k], type_map, ntr[:, s], nt=nt)
                ga3.append(a), ge3.append(e)
            if g2[k] is None or n == 0:
                ga2.append(None), ge2.append(None)
            else:
                a, e = ops.compute_two_body_par_grad(g2[k].contiguous(), rad[:, s], im2[:, s], a2[k], e2[k], type_map)
                ga2.append(a), ge2.append(e)
        return (None, None, None, None, *ga3, *ge3, *ga2, *ge2)


def _type_now(x, device):
    return x if torch.is_tensor(x) else torch.tensor([int(x)], dtype=torch.int32, device=device)


class descriptor_layer(torch.nn.Module):
    """STAF/source_routine/descriptor_builder.py:15-37: configures the descriptor op once, then maps (pos, box) to
    [raddescr, angdescr, des3bsupp, intmap2b, intmap3b, intder2b, intder3b, intder3bsupp, numtriplet]."""

    def __init__(self, rc, rad_buff, rc_ang, ang_buff, N, box_example, Rs, maxbatch, dtype=None):
        super().__init__()
        self.rc, self.rad_buff, self.rc_ang, self.ang_buff, self.N, self.Rs = rc, rad_buff, rc_ang, ang_buff, N, Rs
        self.box_example = box_example
        ops.construct_descriptors_light(rc, rad_buff, ang_buff, N, box_example, Rs, rc_ang, maxbatch,
                                        dtype=dtype if dtype is not None else box_example.dtype)

    def forward(self, pos, box):
        with torch.no_grad():
            rad, ang, sup, im2, im3, d2, d3, d3s, ntr = ops.compute_descriptors_light(pos, box)
        return [rad, ang, sup, im2, im3, d2, d3, d3s, ntr]


class physics_layer(torch.nn.Module):
    """STAF/source_routine/physics_layer_mod.py:9-45: holds alpha2b [nt,Ar], alpha3b [ntc,3Aa] and the (unsquared)
    type embeddings of one centre species; the call returns the fingerprints [nf, Nl, Ar+Aa]."""

    def __init__(self, init_alpha2b, init_alpha3b, initial_type_emb):
        super().__init__()
        P = lambda a: torch.nn.Parameter(torch.as_tensor(a).clone())
        self.alpha2b = P(init_alpha2b)
        self.alpha3b = P(init_alpha3b)
        self.type_emb_2b = P(initial_type_emb[0])
        self.type_emb_3b = P(initial_type_emb[1])
        self.nalpha_r = self.alpha2b.shape[1]
        self.nalpha_a = self.alpha3b.shape[1] // 3
        self.output_dim = self.nalpha_r + self.nalpha_a

    def forward(self, x2b, x3bsupp, intmap2b, x3b, intmap3b, numtriplet, type_map):
        emb2 = torch.square(self.type_emb_2b)
        emb3 = torch.square(self.type_emb_3b)
        af2 = _SortProj.apply(x2b, intmap2b, self.alpha2b, emb2, type_map)
        af3 = _SortProj3body.apply(x3b, x3bsupp, intmap3b, intmap2b, self.alpha3b, emb3, type_map, numtriplet)
        return torch.cat([af2, af3], dim=2)

    def savealphas(self, folder_ou, prefix):
        """The six text files of physics_layer_mod.py:47-53."""
        import numpy as np
        g = lambda t: t.detach().cpu().numpy()
        np.savetxt(f"{folder_ou}/{prefix}alpha_2body.dat", g(self.alpha2b))
        np.savetxt(f"{folder_ou}/{prefix}alpha_3body.dat", g(self.alpha3b))
        np.savetxt(f"{folder_ou}/{prefix}type_emb_2b.dat", g(self.type_emb_2b))
        np.savetxt(f"{folder_ou}/{prefix}type_emb_3b.dat", g(self.type_emb_3b))
        np.savetxt(f"{folder_ou}/{prefix}type_emb_2b_sq.dat", g(self.type_emb_2b) ** 2)
        np.savetxt(f"{folder_ou}/{prefix}type_emb_3b_sq.dat", g(self.type_emb_3b) ** 2)


class descriptor_physics_layer(torch.nn.Module):
    """descriptor_layer followed by the physics_layer of every centre species, as one launch (no counterpart as one
    layer in the reference): `descriptors` is a descriptor_layer (it has configured the descriptor op), `physics` the
    physics_layer modules of the species in species order, `n_local` the atoms per species (species-sorted atoms).
    The call returns what descriptors(pos, box) returns and, per species, what its physics_layer returns for the
    species' rows, with the same bits and the same gradients."""

    def __init__(self, descriptors, physics, n_local):
        super().__init__()
        self.descriptors = descriptors
        self.physics = torch.nn.ModuleList(physics)
        self.n_local = [int(n) for n in n_local]

    def forward(self, pos, box, type_map):
        nt = len(self.n_local)
        params = ([p.alpha3b for p in self.physics] + [torch.square(p.type_emb_3b) for p in self.physics] +
                  [p.alpha2b for p in self.physics] + [torch.square(p.type_emb_2b) for p in self.physics])
        out = _DescriptorsFingerprints.apply(pos, box, type_map, self.n_local, *params)
        desc, af3, af2 = list(out[:9]), out[9:9 + nt], out[9 + nt:9 + 2 * nt]
        return desc, [torch.cat([af2[k], af3[k]], dim=2) for k in range(nt)]


class lognorm_layer(torch.nn.Module):
    """physics_layer_mod.py:54-62: log(AF + 1e-3) - mu with trainable mu."""

    def __init__(self, mu):
        super().__init__()
        self.mu = torch.nn.Parameter(torch.as_tensor(mu).clone())

    def forward(self, restot):
        return torch.log(restot + 1e-3) - self.mu

    def savemu(self, folder_ou, prefix):
        import numpy as np
        np.savetxt(f"{folder_ou}/{prefix}alpha_mu.dat", self.mu.detach().cpu().numpy())


class force_layer(torch.nn.Module):
    """force_layer_mod.py:8-44: 2-body + 3-body forces of one centre species from dE/dAF (net_der_r, net_der_a)."""

    def __init__(self, radbuff, angbuff):
        super().__init__()
        ops.init_force_radial(radbuff)
        ops.init_force_tripl(angbuff)
        ops.init_grad_force_radial(radbuff)
        ops.init_grad_force_tripl(angbuff)

    def forward(self, net_der_r, x2b, intder2b, int2b, alpha2b, net_der_a, x3b, x3bsupp, intder3b, intder3bsupp, int3b,
                numtriplet, alpha3b, type_emb_2b, type_emb_3b, type_map, tipos, type_now):
        tn = _type_now(type_now, x2b.device)
        f2 = _ForceRadial.apply(net_der_r, intder2b, int2b, x2b, alpha2b, torch.square(type_emb_2b), type_map, tipos,
                                tn, None, None)
        f3 = _ForceTripl.apply(net_der_a, x3bsupp, x3b, intder3bsupp, intder3b, int2b, int3b, alpha3b,
                               torch.square(type_emb_3b), type_map, tipos, tn, numtriplet, None, None)
        return f2 + f3


class force_virial_layer(torch.nn.Module):
    """force_layer_mod.py:75-103: forces and the full virial tensor [nf, 9]."""

    def __init__(self, radbuff, angbuff, with_grad=True):
        super().__init__()
        ops.init_force_radial(radbuff)
        ops.init_force_tripl(angbuff)
        if with_grad:
            ops.init_grad_force_radial(radbuff)
            ops.init_grad_force_tripl(angbuff)

    def forward(self, net_der_r, x2b, intder2b, int2b, alpha2b, net_der_a, x3b, x3bsupp, intder3b, intder3bsupp, int3b,
                numtriplet, alpha3b, type_emb_2b, type_emb_3b, type_map, tipos, type_now, pos, box):
        tn = _type_now(type_now, x2b.device)
        f2, w2 = _ForceRadial.apply(net_der_r, intder2b, int2b, x2b, alpha2b, torch.square(type_emb_2b), type_map,
                                    tipos, tn, pos, box)
        f3, w3 = _ForceTripl.apply(net_der_a, x3bsupp, x3b, intder3bsupp, intder3b, int2b, int3b, alpha3b,
                                   torch.square(type_emb_3b), type_map, tipos, tn, numtriplet, pos, box)
        return f2 + f3, w2 + w3
