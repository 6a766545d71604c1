"""Inputs that put atoms exactly on the periodic box faces, shared by the CPU oracle tests and the GPU
parity tests of the neighbour search.

The reference wraps a coordinate as remainderf(x - box/2, box) + box/2
(extensions/neighbour_grid/neighbour_grid_kern.cu:39-42,75-76).  IEEE remainder rounds the quotient
to nearest even, so x = box, -box, 3 box, ... and x within half an ulp below box all wrap to exactly
`box`, not 0; the cell index (int)(ndiv*w/box) % ndiv (:78-80) then files such an atom in cell 0
while its coordinate is `box`.  Its partners in cell 1 are found only through the +-box of the
minimum image (:44-48), which the reference applies to every pair.
"""
import numpy as np

FACE_BOXES = [((70., 70., 70.), 6.0), ((86.861, 86.861, 86.861), 6.0), ((55., 55., 55.), 5.0),
              ((30.5, 33.5, 36.5), 7.0)]


def face_values(box_len):
    b = np.float32(box_len)
    return np.array([b, -b, np.nextafter(b, np.float32(0)), 0.0, 3 * b, 2 * b, -2 * b, np.nextafter(-b, np.float32(0)),
                     np.nextafter(np.float32(0), np.float32(1)), -np.nextafter(np.float32(0), np.float32(1))],
                    dtype=np.float32)


def hand_placed_line(box, cutoff, axis):
    """Pairs (face atom, partner) along one axis: the face atom's coordinate wraps to `box` or 0, the
    partner sits in the next cell (cell 1) within the cutoff of the face, and symmetrically in the last
    cells.  Other coordinates are spread so that different pairs do not see each other."""
    L = np.float32(box[axis])
    nd = int(np.ceil(np.float32(L) / np.float32(cutoff)))
    width = L / nd
    pts = []
    other = 0
    for f in face_values(L):
        for frac in (1.001, 0.5 * (1 + cutoff / width), 0.999 * cutoff / width):     # inside cell 1, below the cutoff
            if frac * width > cutoff or frac < 1.0:
                continue
            for sign in (+1, -1):
                a = np.zeros(3, dtype=np.float32)
                b = np.zeros(3, dtype=np.float32)
                off = np.float32(2.5 * cutoff * (other % 3) + 1.0)
                off2 = np.float32(2.5 * cutoff * ((other // 3) % 3) + 1.0)
                a[axis] = f
                b[axis] = np.float32(sign * frac * width) if sign > 0 else np.float32(L - frac * width)
                for p in (a, b):
                    p[(axis + 1) % 3] = off
                    p[(axis + 2) % 3] = off2
                pts += [a, b]
                other += 1
    return np.stack(pts)[None].astype(np.float32)


def snapped_random(box, n_atoms, batch, seed, frac=0.05):
    """Uniform atoms (also outside the box) with `frac` of all coordinates snapped to face values."""
    rng = np.random.default_rng(seed)
    bx = np.array(box, dtype=np.float32)
    x = ((rng.random((batch, n_atoms, 3)) * 3 - 1) * bx).astype(np.float32)
    for d in range(3):
        vals = face_values(bx[d])
        hit = rng.random((batch, n_atoms)) < frac
        x[..., d][hit] = vals[rng.integers(0, len(vals), hit.sum())]
    return x
