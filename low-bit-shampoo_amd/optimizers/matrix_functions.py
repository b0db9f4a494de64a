"""Inverse p-th roots of PSD matrices by the coupled Newton iteration.

Same three entry points, argument meaning and return values as the reference's
optimizers/matrix_functions.py (PowerIter :21-48, MatPower :51-76, ComputePower :79-141); they
accept CPU or GPU tensors and then behave like the reference, sync for sync.

ComputePowerBatched is the MI355X form of ComputePower for a whole stack of equally sized
matrices: every product runs on the matrix cores through qtensor.fused.gemm (4 launches per
iteration for the whole stack), max|M - I| and the next iteration matrix come out of the last
product's epilogue, and the per-matrix stopping rules are evaluated on the device, so the host
never waits inside the iteration.
"""
from typing import Optional

import torch


@torch.no_grad()
def PowerIter(mat_g, error_tolerance=1e-6, num_iters=10, v0=None):
    """Largest eigenvalue of a symmetric PSD matrix by at most num_iters normalised
    matrix-vector products, starting from v0 (default: uniform in (-1, 1), drawn on mat_g's
    device from the global generator).  Stops once the Rayleigh quotient moves by no more than
    error_tolerance.  Returns (eigenvalue, unit vector, iterations used)."""
    n = mat_g.shape[0]
    v = torch.rand(n, device=mat_g.device) * 2 - 1 if v0 is None else v0.to(mat_g.device)
    change, used, value = 1, 0, 0
    while change > error_tolerance and used < num_iters:
        v = v / torch.norm(v)
        w = torch.mv(mat_g, v)
        quotient = torch.dot(v, w)
        change = torch.abs(quotient - value)
        v, value = w, quotient
        used += 1
    return value, v / torch.norm(v), used


@torch.no_grad()
def MatPower(mat_m, p):
    """mat_m ** p for a positive integer p: repeated squaring for powers of two up to 32,
    square-and-multiply otherwise."""
    if p in (1, 2, 4, 8, 16, 32):
        out, done = mat_m, 1
        while done < p:
            out = torch.matmul(out, out)
            done *= 2
        return out
    result, base = None, mat_m
    while p > 0:
        if p & 1:
            result = base if result is None else torch.matmul(base, result)
        p >>= 1
        base = torch.matmul(base, base)
    return result


@torch.no_grad()
def ComputePower(mat_g, p, iter_count=10, error_tolerance=1e-6, ridge_epsilon=1e-6, v0=None):
    """(mat_g + r I)^(-1/p), r = ridge_epsilon * (largest eigenvalue estimate), by the coupled
    Newton iteration of Guo & Higham (SIAM J. Matrix Anal. Appl. 28(3), 2006, eq. 3.2).

    A vector argument is treated as a diagonal: (mat_g + ridge_epsilon)^(-1/p) elementwise.
    A 1 x 1 matrix returns the identity.  Like the reference, the ridge is added to mat_g IN
    PLACE.  The iteration stops when max|M - I| <= error_tolerance, after iter_count rounds, or
    when that error grows by more than 20 % (the previous iterate is then returned)."""
    if mat_g.dim() == 1:
        return torch.pow(mat_g + ridge_epsilon, -1 / p)
    n = mat_g.shape[0]
    eye = torch.eye(n, device=mat_g.device)
    if n == 1:
        return eye
    w = -1.0 / p
    top, _, _ = PowerIter(mat_g, v0=v0)
    mat_g += (ridge_epsilon * top) * eye
    z = (1 + p) / (2 * torch.norm(mat_g))
    root = eye * torch.pow(z, 1.0 / p)
    m = mat_g * z
    err = torch.max(torch.abs(m - eye))
    rounds = 0
    while err > error_tolerance and rounds < iter_count:
        t = (1 - w) * eye + w * m
        candidate = torch.matmul(root, t)
        m = torch.matmul(MatPower(t, p), m)
        new_err = torch.max(torch.abs(m - eye))
        if new_err > err * 1.2:
            break
        root, err = candidate, new_err
        rounds += 1
    return root


_LAST_ROUNDS = {}                                  # order -> int32 [B], for diagnostics


@torch.no_grad()
def PowerIterBatched(mats, error_tolerance=1e-6, num_iters=10, v0=None):
    """PowerIter for a stack [B, n, n]; every matrix follows its own stopping rule (entries that
    have converged are frozen).  v0: optional [B, n] or [n] start vectors.  Returns the [B]
    eigenvalue estimates.  No host synchronisation."""
    from qtensor import fused as X
    B, n, _ = mats.shape
    if v0 is None:
        v = torch.rand(B, n, device=mats.device) * 2 - 1
    else:
        v = v0.to(mats.device).expand(B, n).clone()
    value = torch.zeros(B, device=mats.device)
    change = torch.ones(B, device=mats.device)
    own = X.on_matrix_cores(mats) and mats.is_contiguous()          # the stack-wide matrix-vector kernel of the library
    for _ in range(num_iters):
        active = change > error_tolerance
        u = v / torch.linalg.vector_norm(v, dim=1, keepdim=True)
        w = X.matvec(mats, u.contiguous()) if own else torch.bmm(mats, u.unsqueeze(2)).squeeze(2)
        quotient = (u * w).sum(dim=1)
        change = torch.where(active, (quotient - value).abs(), change)
        value = torch.where(active, quotient, value)
        v = torch.where(active.unsqueeze(1), w, v)
    return value


@torch.no_grad()
def ComputePowerBatched(mats, p=4, iter_count=10, error_tolerance=1e-6, ridge_epsilon=1e-6, v0=None,
                        out: Optional[torch.Tensor] = None, symmetric: bool = False):
    """ComputePower for a GPU stack mats [B, n, n] (fp32, overwritten with mats + ridge like the
    reference does for its argument).  Returns [B, n, n].

    symmetric: the caller guarantees mats[b] == mats[b].T bit for bit.  All iterates are then
    symmetric in exact arithmetic and only their upper halves are multiplied out (half the work).
    A dequantized low-bit statistic is NOT symmetric (every row segment has its own scale), and
    the reference iterates on it as it is: leave the flag off for those."""
    from qtensor import fused as X

    if not mats.is_cuda or mats.dtype != torch.float32 or mats.dim() != 3:
        raise ValueError("ComputePowerBatched takes an fp32 GPU stack [B, n, n]")
    if p not in (1, 2, 4, 8, 16, 32):
        raise ValueError("ComputePowerBatched supports p in 1, 2, 4, ..., 32")
    B, n, _ = mats.shape
    dev = mats.device
    eye = torch.eye(n, device=dev)
    if n == 1:
        res = eye.expand(B, 1, 1).clone()
        return res if out is None else out.copy_(res)
    w = -1.0 / p
    top = PowerIterBatched(mats, v0=v0)
    mats.diagonal(dim1=1, dim2=2).add_((ridge_epsilon * top).unsqueeze(1))
    z = (1 + p) / (2 * torch.linalg.matrix_norm(mats))                       # [B]
    R = [torch.zeros(B, n, n, device=dev), torch.empty(B, n, n, device=dev)]
    first_root = torch.pow(z, 1.0 / p)                                       # the root starts as this multiple of the identity
    R[0].diagonal(dim1=1, dim2=2).copy_(first_root.unsqueeze(1).expand(B, n))
    M = [mats * z.view(B, 1, 1), torch.empty(B, n, n, device=dev)]
    T = [(1 - w) * eye + w * M[0], torch.empty(B, n, n, device=dev)]
    T2 = torch.empty(B, n, n, device=dev)
    Tp = torch.empty(B, n, n, device=dev)
    err = (M[0] - eye).abs().amax(dim=(1, 2))
    rounds = torch.zeros(B, dtype=torch.int32, device=dev)
    done = (err <= error_tolerance)

    # which of the two buffers currently holds matrix b's accepted R / M / T: pointer tables on
    # the device, swapped per matrix when a round is accepted
    def table(pair):
        step = pair[0].stride(0) * 4
        return [torch.arange(B, device=dev, dtype=torch.int64) * step + t.data_ptr() for t in pair]

    R_ptr, M_ptr, T_ptr = table(R), table(M), table(T)
    side = torch.zeros(B, dtype=torch.bool, device=dev)                     # False: buffer 0 holds the state
    for round_number in range(iter_count):
        skip = done.to(torch.int32)
        cur = lambda tab: torch.where(side, tab[1], tab[0])                   # noqa: E731
        oth = lambda tab: torch.where(side, tab[0], tab[1])                   # noqa: E731
        Rc, Ro, Mc, Mo, Tc, To = cur(R_ptr), oth(R_ptr), cur(M_ptr), oth(M_ptr), cur(T_ptr), oth(T_ptr)
        shape = (B, n, n)
        if round_number == 0:
            # candidate root of the first round: (c I) T = c T, every matrix still in its first buffer
            torch.mul(T[0], first_root.view(B, 1, 1), out=R[1])
        else:
            X.gemm(X.PtrList(Rc, shape), X.PtrList(Tc, shape), out=X.PtrList(Ro, shape), skip=skip,
                   symmetric=symmetric)                                      # candidate root
        power = X.PtrList(Tc, shape)                                         # T^p by repeated squaring
        done_p = 1
        while done_p < p:
            dst = Tp if power is T2 else T2
            X.gemm(power, power, out=dst, skip=skip, symmetric=symmetric)
            power, done_p = dst, done_p * 2
        new_err = torch.zeros(B, device=dev)
        X.gemm(power, X.PtrList(Mc, shape), out=X.PtrList(Mo, shape), newton=(X.PtrList(To, shape), w, new_err),
               skip=skip, symmetric=symmetric)
        accept = (~done) & ~(new_err > err * 1.2)
        side = side ^ accept
        err = torch.where(accept, new_err, err)
        rounds = rounds + accept.to(torch.int32)
        done = done | ~accept | (err <= error_tolerance) | (rounds >= iter_count)
    _LAST_ROUNDS[n] = rounds                       # accepted rounds per matrix of the last stack of this order
    res = torch.where(side.view(B, 1, 1), R[1], R[0])
    return res if out is None else out.copy_(res)
