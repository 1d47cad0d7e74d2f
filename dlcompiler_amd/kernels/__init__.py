"""Host-side operator entry points; one module per ``dlblas.kernels`` module mirrored."""
