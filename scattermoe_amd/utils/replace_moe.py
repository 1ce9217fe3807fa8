"""Hugging Face injection (placeholder filled in below)."""
