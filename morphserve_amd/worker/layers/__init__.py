from .transformer_layer import attention_section  # noqa: F401
