"""Host-side helpers around the quantized-linear path (checkpoint conversion)."""
