"""Host-side communication compiler: IR, plan builders, signal planning, op-list generation."""
