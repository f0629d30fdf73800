"""QVB8R: the QVB8 band ids, rANS-coded (32 interleaved streams per tile, 12-bit probabilities)."""
