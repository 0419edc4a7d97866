"""Drop-in surface of the reference's `fsa` package, backed by libfsa_gfx950.so."""
