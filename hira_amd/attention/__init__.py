from .hira_attention import hira_attention_forward, register_hira_attention

__all__ = ["hira_attention_forward", "register_hira_attention"]
