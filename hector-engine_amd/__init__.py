"""Qwen2 dense generation library for one MI355X (package folder ``hector-engine_amd``)."""
