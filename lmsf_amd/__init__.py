"""lmsf_amd: a small, whole LLM inference engine for one MI355X."""
__version__ = "0.1.0"
