"""MI355X-native W4A16 linear op (int4-symmetric weights x f16 activations): host-side mirror of the reference's
operator interface over a C-ABI HIP library.  See llm170_amd.ffi for the binding and llm170_amd.ops for the
operator classes."""
