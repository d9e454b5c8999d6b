# namespace of the torch.library custom ops, the reference's LIBRARY_NAME (fma/constants.py:10)
LIBRARY_NAME = "flash_model_architectures"
