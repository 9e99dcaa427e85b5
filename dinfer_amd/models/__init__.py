from . import fanulix, karopel, kudurax, qwen3  # noqa: F401  (register the built-in architectures)
