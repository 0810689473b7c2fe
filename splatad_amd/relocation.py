"""`compute_relocation` of the reference (`gsplat/relocation.py:10-49`) on the HIP library."""
from typing import Tuple

from torch import Tensor

from .hip._wrapper import _make_lazy_hip_func


def compute_relocation(
    opacities: Tensor,  # [N]
    scales: Tensor,  # [N, 3]
    ratios: Tensor,  # [N]
    binoms: Tensor,  # [n_max, n_max]
) -> Tuple[Tensor, Tensor]:
    """Opacities and scales of the copies when every Gaussian is split into `ratios[i]` equal
    ones (equation 9 of "3D Gaussian Splatting as Markov Chain Monte Carlo").  `binoms[n, k]`
    holds the binomial coefficients; `ratios` is clamped to [1, n_max] in place, as in the
    reference.  Returns (new_opacities [N], new_scales [N, 3])."""
    N = opacities.shape[0]
    n_max, _ = binoms.shape
    assert scales.shape == (N, 3), scales.shape
    assert ratios.shape == (N,), ratios.shape
    opacities = opacities.contiguous()
    scales = scales.contiguous()
    ratios.clamp_(min=1, max=n_max)
    ratios = ratios.int().contiguous()
    return _make_lazy_hip_func("compute_relocation")(opacities, scales, ratios, binoms.contiguous(), n_max)
