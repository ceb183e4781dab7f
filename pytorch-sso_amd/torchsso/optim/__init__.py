from torchsso.optim.secondorder import SecondOrderOptimizer  # NOQA
from torchsso.optim.vi import VIOptimizer, VOGN  # NOQA
