from var_q_amd.config_loader import *  # noqa: F401,F403
from var_q_amd.config_loader import VARQConfig, load_varq_config  # noqa: F401
