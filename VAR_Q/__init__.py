"""Import-name alias of the reference package: `from VAR_Q.quant import VAR_Q`,
`from VAR_Q.pack_unpack import ...`, `from VAR_Q.config_loader import ...` resolve
to the MI355X implementation in `var_q_amd`."""
