"""Runtime side of the communication compiler: op records and the single-GPU executor."""
