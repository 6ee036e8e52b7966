from .deit_dge import *  # noqa: F401,F403
