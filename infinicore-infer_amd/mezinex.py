"""The entry point under the Mezinex architecture's name: ``MezinexForCausalLM`` and
``python -m infinicore_infer_amd.mezinex``.  Class and command line are the architecture-neutral ones of
``causal_lm``; which model is built is decided by config.json through the architecture registry.
"""
from .causal_lm import DEVICE_FLAGS, USAGE, CausalLM, test      # noqa: F401

MezinexForCausalLM = CausalLM


if __name__ == "__main__":
    test()
