"""Test infrastructure only: CPU restatement of the reference's GPTQ path.  Never imported by moe_quant_amd."""
