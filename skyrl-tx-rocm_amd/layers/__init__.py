"""Module-level mirror of the reference's LoRA layers on the W8A8 path."""
