"""The engine: step function, scheduler, request loop, replay."""
