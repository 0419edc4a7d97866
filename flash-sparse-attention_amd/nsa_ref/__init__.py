"""Drop-in surface of the reference's `nsa_ref` package for the operators the FSA layer uses."""
