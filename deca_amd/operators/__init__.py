from .Op import *  # noqa: F401,F403
from .GEMMTC import *  # noqa: F401,F403
from .FlashAttention import *  # noqa: F401,F403
from .Rowwise import *  # noqa: F401,F403
from .Softmax import *  # noqa: F401,F403
from .RMSNorm import *  # noqa: F401,F403
