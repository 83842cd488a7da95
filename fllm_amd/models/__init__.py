from . import dumizen, llama, menitar, purivik, venadra  # noqa: F401  (register the architectures)
