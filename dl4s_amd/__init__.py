"""dl4s_amd: MI355X (gfx950) backend for the attention forward path of DL4S.

`dl4s_amd.lib` binds the C ABI of libdl4s_hip.so; `dl4s_amd.build` compiles it.
"""
