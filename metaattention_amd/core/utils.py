"""Small host-side helpers of the public API."""


class meta_tensor:
    """Shape + dtype holder users describe q/k/v with
    (``meta_tensor(B, H, S, D, dtype=torch.bfloat16)``), as in the reference's
    core/utils.py:40-47."""

    def __init__(self, *shape, **kwargs):
        self.shape = shape
        self.kargs = kwargs

    @property
    def dtype(self):
        return self.kargs["dtype"]

    def __repr__(self):
        return f"meta_tensor{self.shape}, dtype={self.kargs.get('dtype')}"
