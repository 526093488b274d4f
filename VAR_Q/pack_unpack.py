from var_q_amd.pack_unpack import *  # noqa: F401,F403
