from . import llama, menitar  # noqa: F401  (register the architectures)
