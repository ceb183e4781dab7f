from torchsso.utils.linalg import inv, cholesky  # NOQA
from torchsso.utils.accumulator import TensorAccumulator  # NOQA
from torchsso.utils.packer import Packer  # NOQA
