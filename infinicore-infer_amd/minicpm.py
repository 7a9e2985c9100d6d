"""The entry point under the architecture's own name, as the reference names its script after its model
(scripts/jiuge.py): ``MiniCPMForCausalLM`` and ``python -m infinicore_infer_amd.minicpm``.  Class and
command line are the architecture-neutral ones of ``causal_lm``; which model is built is decided by
config.json through the architecture registry.
"""
from .causal_lm import DEVICE_FLAGS, USAGE, CausalLM, test      # noqa: F401

MiniCPMForCausalLM = CausalLM


if __name__ == "__main__":
    test()
