"""Graph front-end for the planner harness: model definitions that give the
benchmark graphs their shape, joint forward+backward capture on fake tensors, and
strategy enumeration over a logical mesh."""
