"""Text on either side of the token ids: tokenizers of a model folder and the piecewise decoder
of generated tokens.  Used by the server layer and the command line; the engine never sees text."""
