"""Test infrastructure: CPU restatement of the reference's naive NSA forward path."""
