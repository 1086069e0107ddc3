"""Run-time half of the scheduling layer: environment, engine, device seam."""
