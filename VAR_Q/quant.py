from var_q_amd.quant import *  # noqa: F401,F403
from var_q_amd.quant import VAR_Q  # noqa: F401
