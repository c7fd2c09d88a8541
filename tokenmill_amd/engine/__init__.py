"""The engine: step function, scheduler, request records and the generation loop."""
