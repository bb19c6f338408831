from .moe_permute import *  # noqa: F401,F403
