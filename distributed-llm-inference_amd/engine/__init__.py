"""Step function, scheduler and the engine's Python entry points."""
