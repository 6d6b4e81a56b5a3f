"""Hugging Face plug-in boundary."""
