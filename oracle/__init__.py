"""CPU oracle for the GGUF quantized-linear path: test infrastructure, never imported by tur_amd."""
