"""Fill / Generate primitives as the engine's iteration loop sees them
(parrot/engine/primitive_job.py:13-125): ids, the bound context, the finish
event, and for Generate the token stream and stop conditions."""
from __future__ import annotations

import collections
import threading
from typing import Any, Deque, List, Optional


class PrimitiveJob:
    def __init__(self, session_id: int, task_id: int, context_id: int, parent_context_id: int, end_flag: bool = False):
        self.session_id = session_id
        self.task_id = task_id
        self.context_id = context_id
        self.parent_context_id = parent_context_id
        self.end_flag = end_flag
        self.context = None  # BlockContext, bound by the engine
        self.finish_event = threading.Event()
        self.start_time: float = -1
        self.end_time: float = -1


class Fill(PrimitiveJob):
    def __init__(self, session_id: int, task_id: int, context_id: int, parent_context_id: int, end_flag: bool = False,
                 token_ids: Optional[List[int]] = None, text: Optional[str] = None):
        super().__init__(session_id, task_id, context_id, parent_context_id, end_flag)
        self.token_ids = token_ids
        self.text = text

    def __repr__(self) -> str:
        return (f"Fill(session_id={self.session_id}, task_id={self.task_id}, context_id={self.context_id}, "
                f"parent_context_id={self.parent_context_id})")


class Generate(PrimitiveJob):
    def __init__(self, session_id: int, task_id: int, context_id: int, parent_context_id: int,
                 sampling_config: Any = None, end_flag: bool = False):
        super().__init__(session_id, task_id, context_id, parent_context_id, end_flag)
        self.sampling_config = sampling_config
        self.output_queue: Deque[int] = collections.deque()  # token stream
        self.gen_text = ""
        self.gen_length = 0

    def __repr__(self) -> str:
        return (f"Generate(session_id={self.session_id}, task_id={self.task_id}, context_id={self.context_id}, "
                f"parent_context_id={self.parent_context_id})")

    def put_token(self, token_id: int) -> None:
        self.output_queue.append(token_id)
        self.context.push_token_id(token_id)
        self.gen_length += 1

    def check_stop(self) -> bool:
        token_id = self.context.get_last_token_id()
        sc = self.sampling_config
        return token_id in sc.stop_token_ids or self.gen_length >= sc.max_gen_length
