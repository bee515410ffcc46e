"""CPU restatements of the reference codec, used only as checkers by tests, smoke and the CPU-baseline bench leg."""
