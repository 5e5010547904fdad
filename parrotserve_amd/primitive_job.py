"""Fill / Generate primitives as the attention path sees them
(parrot/engine/primitive_job.py:15-100): only the fields the hot path reads."""
from __future__ import annotations

from typing import Any, List, Optional


class PrimitiveJob:
    def __init__(self, session_id: int, task_id: int, context_id: int, parent_context_id: int, end_flag: bool = False):
        self.session_id = session_id
        self.task_id = task_id
        self.context_id = context_id
        self.parent_context_id = parent_context_id
        self.end_flag = end_flag
        self.context = None  # BlockContext, bound by the engine


class Fill(PrimitiveJob):
    def __init__(self, session_id: int, task_id: int, context_id: int, parent_context_id: int, end_flag: bool = False,
                 token_ids: Optional[List[int]] = None, text: Optional[str] = None):
        super().__init__(session_id, task_id, context_id, parent_context_id, end_flag)
        self.token_ids = token_ids
        self.text = text


class Generate(PrimitiveJob):
    def __init__(self, session_id: int, task_id: int, context_id: int, parent_context_id: int,
                 sampling_config: Any = None, end_flag: bool = False):
        super().__init__(session_id, task_id, context_id, parent_context_id, end_flag)
        self.sampling_config = sampling_config
