"""Drop-in surface of the reference's `fsa_preview` decode operators."""
