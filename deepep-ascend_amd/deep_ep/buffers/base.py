from abc import ABC, abstractmethod


class BufferBase(ABC):
    """Lifecycle shared by the communication buffers: a native runtime object that is either
    destroyed explicitly or with its owner."""

    def __init__(self, explicitly_destroy: bool = False):
        self.explicitly_destroy = explicitly_destroy
        self.runtime = None

    @property
    def main_context(self):
        return None if self.runtime is None else self.runtime.main_context

    def print_memory_usage(self) -> None:
        assert self.runtime is not None
        self.runtime.print_memory_usage()

    @abstractmethod
    def destroy(self) -> None:
        assert self.explicitly_destroy
        runtime, self.runtime = self.runtime, None
        if runtime is not None:
            runtime.destroy()
