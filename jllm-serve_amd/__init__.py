"""An inference engine for one AMD Instinct MI355X: model folder in, token ids out.

config/    typed configuration and the architecture registry
weights/   safetensors reader/writer, by-name loader, random-weights mode
parts/     mixers, feed-forwards, norms, position encodings, their arrangement, the decoder model
cache/     pages, block tables per request and layer group, state slots
engine/    the step function, the scheduler, generation, trace replay
sampling/  sampling parameters and the sampler
kernels/   Python faces of the HIP kernels under csrc/ and their in-tree build
"""
__version__ = "0.1.0"
