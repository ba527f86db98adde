import torch

from . import classes


class CubicSpline(torch.nn.Module):
    """Natural cubic spline through (r_knots[k], R_out[k, :]), evaluated per edge on the GPU.

    Same constructor and buffers as the reference (ops/cubic_spline.py:4-39): r_knots [K], R_out [K, J],
    knot spacing h, cutoff rmax; buffer `coefficients` [K-1, 4, J] holds (a, b, c, d) of
    a + b x + c x^2 + d x^3 with x = r - r_knots[k].  forward(r [nedges]) -> [nedges, J]; zero for r > rmax.
    """

    def __init__(self, r_knots: torch.Tensor, R_out: torch.Tensor, h: float, rmax: float):
        super().__init__()
        self.register_buffer("r_knots", r_knots)
        self.register_buffer("R_out", R_out)
        self.register_buffer("h", torch.tensor(float(h), device=r_knots.device))
        self.register_buffer("rmax", torch.tensor(float(rmax), device=r_knots.device))
        self._h = float(h)
        self._rmax = float(rmax)
        coefficients = self.cubic_spline_coefficients(self.r_knots, self.R_out, self._h)
        self.register_buffer("coefficients", coefficients.to(R_out.dtype).contiguous())
        self.cuda_obj = classes.cubic_spline.CubicSpline()

    def forward(self, r_trial: torch.Tensor):
        return self.cuda_obj.forward(r_trial, self.r_knots, self.coefficients, self._h, self._rmax)

    @staticmethod
    def cubic_spline_coefficients(x: torch.Tensor, y: torch.Tensor, h: float) -> torch.Tensor:
        """Textbook natural-spline solve (second derivative zero at both ends) on a uniform grid, all
        columns of y at once, in fp64.  Same result as the reference's per-knot Python loops
        (ops/cubic_spline.py:41-84): tridiagonal system for the second-order coefficients c, then b, d."""
        yd = y.double()
        n = x.shape[0] - 1
        J = yd.shape[1]
        alpha = torch.zeros(n + 1, J, dtype=torch.float64, device=y.device)
        alpha[1:n] = 3.0 / h * (yd[2:] - 2.0 * yd[1:-1] + yd[:-2])
        # Thomas algorithm for h c[i-1] + 4h c[i] + h c[i+1] = alpha[i], c[0] = c[n] = 0
        mu = torch.zeros(n + 1, dtype=torch.float64)
        z = torch.zeros(n + 1, J, dtype=torch.float64, device=y.device)
        for i in range(1, n):
            li = 4.0 * h - h * float(mu[i - 1])
            mu[i] = h / li
            z[i] = (alpha[i] - h * z[i - 1]) / li
        c = torch.zeros(n + 1, J, dtype=torch.float64, device=y.device)
        for j in range(n - 1, -1, -1):
            c[j] = z[j] - float(mu[j]) * c[j + 1]
        b = (yd[1:] - yd[:-1]) / h - h * (c[1:] + 2.0 * c[:-1]) / 3.0
        d = (c[1:] - c[:-1]) / (3.0 * h)
        return torch.stack((yd[:-1], b, c[:-1], d), dim=1)
