"""Quantization formats, codecs, transforms and algorithms of the packed-inference path."""
