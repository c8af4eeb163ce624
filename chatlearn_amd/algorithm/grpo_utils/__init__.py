"""Drop-in mirrors of chatlearn/algorithm/grpo_utils (same names, signatures and
return types), computing on the GPU through libclgrpo.so."""
