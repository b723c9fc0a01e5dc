"""CPU oracle of the quantized TorqHL operator path (test infrastructure only)."""
