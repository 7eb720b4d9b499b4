"""Engine: model assembly, the step function, generation and trace replay."""
