from . import fanulix, karopel, kudurax, qwen3, verorax  # noqa: F401  (register the built-in architectures)
