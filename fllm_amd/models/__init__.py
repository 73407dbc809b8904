from . import llama, menitar, purivik  # noqa: F401  (register the architectures)
