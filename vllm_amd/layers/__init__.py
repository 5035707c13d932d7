"""Host-side mirror of the reference's linear-layer plugin surface for the quantized-linear path."""
