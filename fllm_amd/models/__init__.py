from . import llama, menitar, purivik, venadra  # noqa: F401  (register the architectures)
