"""MI355X-native decode path for T5.1.1 encoder-decoder models.

Drop-in for the autoregressive decode path of google-research/t5x:
`t5x_amd.decoding` (beam_search, temperature_sample and helpers),
`t5x_amd.models.EncoderDecoderModel.predict_batch[_with_aux]`, and
`t5x_amd.network.Transformer` (the decoder's single-step forward on
hand-written HIP kernels, bound through the C ABI in include/t5d.h).
"""

__version__ = '0.1.0'
