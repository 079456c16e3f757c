"""Oracle for bitfield-masked attention: test infrastructure, never imported by the shipped package."""
