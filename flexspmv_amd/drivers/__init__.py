"""Models that call the fused path, written against :mod:`flexspmv_amd.frontend` the way the reference's
drivers are written against EASIER, plus the original-versus-replaced check that exercises them."""
