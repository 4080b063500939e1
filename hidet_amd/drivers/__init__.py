from .build_task import build_task_library
