"""The part of the reference's `glm53f-forward` crate that saves and restores a slot's positional state
(KDA states, conv windows, tails) in pages of the KV pool: the byte layout and page accounting
(`kvplan`, crates/glm53f-forward/src/kvplan.rs), the raw bindings of the row gather/scatter
(`ffi`, crates/glm53f-forward/src/ffi.rs:75-96) and the device side of marks (`kv`,
crates/glm53f-forward/src/kv.rs:385-560, :575-720). There is no CPU fallback: the copies are the HIP library's.
"""
