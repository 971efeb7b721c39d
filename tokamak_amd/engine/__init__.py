"""Engine: model assembly, step function, scheduler, generation loop."""
