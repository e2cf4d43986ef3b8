"""dhellam.adaptor.megatron: the Megatron-LM initialisation is outside the single-GPU operator path."""


def initialize_dhellam_megatron(*args, **kwargs):
    raise RuntimeError("initialize_dhellam_megatron needs Megatron-LM and a process group; this build covers the "
                       "per-rank operator path on one GPU (see dhellam_amd.core.layer / dhellam_amd.core.dsllm)")
