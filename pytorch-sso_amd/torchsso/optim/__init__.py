from torchsso.optim.secondorder import SecondOrderOptimizer  # NOQA
from torchsso.optim.vi import VIOptimizer, VOGN  # NOQA
from torchsso.optim import lr_scheduler  # NOQA
