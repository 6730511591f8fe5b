"""CPU oracle for the trellis decoders: test infrastructure, never the product path."""
