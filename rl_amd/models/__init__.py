"""Mirrors of the policy-worker post-processors that sit directly on the logprob kernels."""


def _need_single_gpu(cp_size, what: str) -> None:
    if cp_size is not None and int(cp_size) > 1:
        raise NotImplementedError(f"{what}: context parallelism (cp_size={cp_size}) needs more than one GPU")
