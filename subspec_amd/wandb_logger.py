"""Process-wide metrics store with the reference's ``wandb_logger`` interface
(specdecodes/models/utils/wandb_logger.py:4-39): ``log_data`` (exported per generation),
``internal_data`` (running accumulators) and ``flags``."""
from threading import Lock
from typing import Any, Dict


class WandbLogger:
    _instance = None
    _lock = Lock()

    def __new__(cls):
        with cls._lock:
            if cls._instance is None:
                inst = super().__new__(cls)
                inst.log_data: Dict[str, Any] = {}
                inst.flags: Dict[str, Any] = {}
                inst.internal_data: Dict[str, Any] = {}
                cls._instance = inst
        return cls._instance

    def set_flag(self, key: str, value: Any) -> None:
        self.flags[key] = value

    def set_flags(self, **kwargs: Any) -> None:
        self.flags.update(kwargs)

    def get_flag(self, key: str, default: Any = None) -> Any:
        return self.flags.get(key, default)

    def clear_log_data(self) -> None:
        self.log_data.clear()
        self.internal_data.clear()

    def clear_flags(self) -> None:
        self.flags.clear()

    def clear_internal_data(self) -> None:
        self.internal_data.clear()


wandb_logger = WandbLogger()
