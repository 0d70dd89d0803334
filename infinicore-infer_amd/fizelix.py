"""The entry point under the Fizelix architecture's name: ``FizelixForCausalLM`` and
``python -m infinicore_infer_amd.fizelix``.  Class and command line are the architecture-neutral ones of
``causal_lm``; which model is built is decided by config.json through the architecture registry.
"""
from .causal_lm import DEVICE_FLAGS, USAGE, CausalLM, test      # noqa: F401

FizelixForCausalLM = CausalLM


if __name__ == "__main__":
    test()
