"""Prime sets used by the tests (kept in the package so that users get the reference's parameter sets too)."""
from ckks_llm_amd.params import *  # noqa: F401,F403
from ckks_llm_amd.params import CFG1_Q, CFG2_Q, CFG3_P, REF_PARAMS, small_primes  # noqa: F401
