from torchsso import _hip, _ops  # NOQA
