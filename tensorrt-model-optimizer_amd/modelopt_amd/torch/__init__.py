"""``modelopt_amd.torch``: the PyTorch-facing surface (``quantization`` and ``export``)."""
