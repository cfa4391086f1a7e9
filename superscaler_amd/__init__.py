"""MI355X-native batched plan evaluator for Aceso-style parallel-training search."""
__all__ = ["opgraph", "profile_db", "tables", "plan", "synth", "evaluator"]
