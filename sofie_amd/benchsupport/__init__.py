"""What the benchmark needs besides the runtime library: the counter-based generator of the synthetic tensors, a writer of
ONNX files, the benchmark configurations as ONNX models, and the step that emits their Sessions and compiles the timing
harness around them.  The tests import the same pieces from here."""
