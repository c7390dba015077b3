"""Backend registration shim (filled in with the backend classes)."""


def register_attention_backends() -> None:
    return None
