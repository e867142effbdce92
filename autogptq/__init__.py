"""Namespace of the MI355X-native GPTQ QuantLinear path; see ``autogptq.tvm_amd``."""
