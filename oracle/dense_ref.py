"""TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT.

Dense "level view" formulation of the operators, used to pin oracle/aprnet_oracle.cpp on tiny APRs
without importing or compiling the reference.  It shares no code with the oracle: everything is
expressed with dense grids and library routines (F.conv3d, max, mean over 2x2x2 blocks).

V_l = dense grid of level l in which a cell holds the value of the particle that covers it
(particles of level <= l, replicated) or, for a cell that is refined further, the mean of the level
l+1 view over the cell's existing children (= the mean-filled tree value).  At the current maximum
level Lc the refined cells hold the "downsampled particles" stored behind the particles.
"""
import numpy as np
import torch
import torch.nn.functional as F


def coords(it):
    """(level, z, x, y) per index for one access (particles or tree), by walking the row tables."""
    n = it.total_number_particles()
    out = np.zeros((n, 4), np.int64)
    for l in range(it.level_min(), it.level_max() + 1):
        for z in range(it.z_num(l)):
            for x in range(it.x_num(l)):
                b = it.begin(l, z, x)
                e = it.end()
                for i in range(b, e):
                    out[i] = (l, z, x, it.y(i))
    return out


class DenseAPR:
    def __init__(self, apr):
        self.apr = apr
        self.pc = coords(apr.iterator())
        self.tc = coords(apr.tree_iterator())
        self.lmax = apr.level_max()
        self.lmin = apr.level_min()

    def n_parts(self, d):
        lc = self.lmax - d
        return int((self.pc[:, 0] <= lc).sum() + (self.tc[:, 0] == lc).sum())

    def tree_offset(self, level):
        return int((self.pc[:, 0] <= level).sum() - (self.tc[:, 0] < level).sum())

    def dims(self, l):
        return self.apr.level_dims(l)

    def views(self, x, d):
        """x: [C, N_d] double.  Returns {level: V_l [C, z, x, y]} for level_min-1 .. Lc."""
        lc = self.lmax - d
        C = x.shape[0]
        V = {}
        z, xx, y = self.dims(lc)
        v = torch.full((C, z, xx, y), float("nan"), dtype=x.dtype)
        for i, (l, pz, px, py) in enumerate(self.pc):
            if l > lc:
                continue
            f = 1 << (lc - l)
            v[:, pz * f:(pz + 1) * f, px * f:(px + 1) * f, py * f:(py + 1) * f] = x[:, i].view(C, 1, 1, 1)
        off = self.tree_offset(lc)
        for t, (l, pz, px, py) in enumerate(self.tc):
            if l == lc:
                v[:, pz, px, py] = x[:, t + off]
        assert not torch.isnan(v).any(), "level view has uncovered cells: the APR is not a partition"
        V[lc] = v
        for l in range(lc - 1, -1, -1):
            z, xx, y = self.dims(l)
            fine = V[l + 1]
            pad = (0, 2 * y - fine.shape[3], 0, 2 * xx - fine.shape[2], 0, 2 * z - fine.shape[1])
            fp = F.pad(fine, pad, value=float("nan"))
            blocks = fp.view(C, z, 2, xx, 2, y, 2).permute(0, 1, 3, 5, 2, 4, 6).reshape(C, z, xx, y, 8)
            V[l] = torch.nanmean(blocks, dim=-1)
        return V

    # ------------------------------------------------------------------------------ operators
    def fill_tree_mean(self, x, d):
        """x: [N_d] -> tree values for all nodes of level < Lc."""
        lc = self.lmax - d
        V = self.views(x[None], d)
        n = int((self.tc[:, 0] < lc).sum())
        out = torch.zeros(n, dtype=x.dtype)
        for t in range(n):
            l, z, xx, y = self.tc[t]
            out[t] = V[int(l)][0, z, xx, y]
        return out

    def outputs(self, d):
        """(feature index, level, z, x, y) of every output position at level delta d."""
        lc = self.lmax - d
        res = [(i, *self.pc[i]) for i in range(len(self.pc)) if self.pc[i, 0] <= lc]
        off = self.tree_offset(lc)
        res += [(t + off, *self.tc[t]) for t in range(len(self.tc)) if self.tc[t, 0] == lc]
        return res

    def conv(self, x, w, d):
        """x: [Cin, N_d]; w: [Cin, S_exp, Cout, kz, kx, ky] (CPU layout).  -> [Cout, N_d]"""
        lc = self.lmax - d
        V = self.views(x, d)
        kz, kx, ky = w.shape[3:]
        out = torch.zeros(w.shape[2], x.shape[1], dtype=x.dtype)
        dense = {}
        for l in range(self.lmin, lc + 1):
            s = min(w.shape[1] - 1, lc - l)
            wl = w[:, s].permute(1, 0, 2, 3, 4).contiguous()
            dense[l] = F.conv3d(V[l][None], wl, padding=((kz - 1) // 2, (kx - 1) // 2, (ky - 1) // 2))[0]
        for idx, l, z, xx, y in self.outputs(d):
            out[:, idx] = dense[int(l)][:, z, xx, y]
        return out

    def maxpool(self, x, d):
        """x: [C, N_d] -> (out [C, N_{d+1}], argmax int64): max over the children of every tree node of
        level Lc-1; first maximum in the order (z, x, y), particles before downsampled particles."""
        lc = self.lmax - d
        n_out = self.n_parts(d + 1)
        out = torch.zeros(x.shape[0], n_out, dtype=x.dtype)
        arg = torch.zeros(x.shape[0], n_out, dtype=torch.int64)
        ncopy = int((self.pc[:, 0] <= lc - 1).sum())
        out[:, :ncopy] = x[:, :ncopy]
        pmap = {tuple(c[1:]): i for i, c in enumerate(self.pc) if c[0] == lc}
        off = self.tree_offset(lc)
        tmap = {tuple(c[1:]): t + off for t, c in enumerate(self.tc) if c[0] == lc}
        ooff = self.tree_offset(lc - 1)
        for t, (l, z, xx, y) in enumerate(self.tc):
            if l != lc - 1:
                continue
            cand = []
            for m in (pmap, tmap):
                for dz in (0, 1):
                    for dx in (0, 1):
                        for dy in (0, 1):
                            k = (2 * z + dz, 2 * xx + dx, 2 * y + dy)
                            if k in m:
                                cand.append(m[k])
            vals = x[:, cand]
            best = vals.argmax(dim=1)           # torch returns the first maximal element
            for c in range(x.shape[0]):
                mx = vals[c].max()
                first = int((vals[c] == mx).nonzero()[0])
                out[c, t + ooff] = mx
                arg[c, t + ooff] = cand[first]
        return out, arg

    def upsample(self, x, d):
        """x: [C, N_d] (d > 0) -> [C, N_{d-1}]"""
        lc = self.lmax - d
        n_out = self.n_parts(d - 1)
        out = torch.zeros(x.shape[0], n_out, dtype=x.dtype)
        ncopy = int((self.pc[:, 0] <= lc).sum())
        out[:, :ncopy] = x[:, :ncopy]
        off = self.tree_offset(lc)
        parent = {tuple(c[1:]): t + off for t, c in enumerate(self.tc) if c[0] == lc}
        for i, (l, z, xx, y) in enumerate(self.pc):
            if l == lc + 1:
                out[:, i] = x[:, parent[(z // 2, xx // 2, y // 2)]]
        ooff = self.tree_offset(lc + 1)
        for t, (l, z, xx, y) in enumerate(self.tc):
            if l == lc + 1:
                out[:, t + ooff] = x[:, parent[(z // 2, xx // 2, y // 2)]]
        return out

    def reconstruct(self, x, d):
        return self.views(x, d)[self.lmax - d]

    def parent_index(self, which, level):
        """brute-force parent tree index for particles (which=0) / tree nodes (which=1) of `level`"""
        tmap = {tuple(c): t for t, c in enumerate(self.tc)}
        src = self.tc if which else self.pc
        out = np.full(len(src), -1, np.int64)
        for i, (l, z, xx, y) in enumerate(src):
            if l == level:
                out[i] = tmap[(l - 1, z // 2, xx // 2, y // 2)]
        return out
