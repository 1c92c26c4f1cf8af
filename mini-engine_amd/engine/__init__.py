"""Request state, scheduler, step function and the engine loop."""
