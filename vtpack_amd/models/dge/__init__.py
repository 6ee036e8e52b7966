from .deit_dge import *  # noqa: F401,F403
from .pvt_dge import *  # noqa: F401,F403
