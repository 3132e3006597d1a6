"""Small tools around the engine (no part of the product path)."""
