"""The entry point under the Fopezen architecture's name: ``FopezenForCausalLM`` and
``python -m infinicore_infer_amd.fopezen``.  Class and command line are the architecture-neutral ones of
``causal_lm``; which model is built is decided by config.json through the architecture registry.
"""
from .causal_lm import DEVICE_FLAGS, USAGE, CausalLM, test      # noqa: F401

FopezenForCausalLM = CausalLM


if __name__ == "__main__":
    test()
