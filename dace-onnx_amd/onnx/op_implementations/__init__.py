from .utils import *  # noqa: F401,F403
from .mi355x_implementations import *  # noqa: F401,F403
