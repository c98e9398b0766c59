from .templates import LLAMA3_INSTRUCT, TEMPLATES, ChatTemplate, FileTokenizer, get_template, tokenize_conversation

__all__ = ["LLAMA3_INSTRUCT", "TEMPLATES", "ChatTemplate", "FileTokenizer", "get_template", "tokenize_conversation"]
