"""torchsso: K-FAC curvature engine for AMD Instinct MI355X (gfx950).

The Python surface is the one of cybertronai/pytorch-sso for the K-FAC path
(SecondOrderOptimizer / VIOptimizer, the Kron*/Diag* curvature classes looked
up by name on this namespace, torchsso.utils.inv / cholesky); the arithmetic
runs in hand-written HIP kernels behind the C ABI of libkfac_hip.so.
"""
from torchsso import _hip, _lanes, _ops  # NOQA
from torchsso import utils  # NOQA

from torchsso.curv.curvature import Curvature, DiagCurvature, KronCurvature  # NOQA
from torchsso.curv.cov.linear import CovLinear, DiagCovLinear, KronCovLinear  # NOQA
from torchsso.curv.cov.conv import CovConv2d, DiagCovConv2d, KronCovConv2d  # NOQA
from torchsso.curv.cov.batchnorm import CovBatchNorm1d, DiagCovBatchNorm1d, CovBatchNorm2d, DiagCovBatchNorm2d  # NOQA

from torchsso.curv.fisher import Fisher, get_closure_for_fisher  # NOQA
from torchsso.curv.fisher import KronFisherLinear, KronFisherConv2d, DiagFisherBatchNorm2d  # NOQA
from torchsso.curv.fisher import DiagFisherLinear, DiagFisherConv2d  # NOQA

from torchsso import optim  # NOQA

# side streams for the factor products (see torchsso._lanes); 0 = caller's stream only
set_factor_streams = _lanes.set_count
factor_streams = _lanes.count
join_factor_streams = _lanes.join
# 'grouped' (default): hooks collect their factor products, the first reader of factor data
# runs them in one engine call; 'eager': every product runs in its hook, on the side streams
set_factor_mode = _lanes.set_mode
factor_mode = _lanes.mode
set_factor_flush_work = _lanes.set_flush_work

__version__ = '0.1.0'
