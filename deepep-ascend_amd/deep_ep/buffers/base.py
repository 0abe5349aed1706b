"""What every communication buffer shares: it owns one native runtime object, and that object is
released either by an explicit `destroy()` or together with its owner (reference:
deep_ep/buffers/base.py, csrc/buffers/base.hpp)."""
import abc


class BufferBase(abc.ABC):
    runtime = None

    def __init__(self, explicitly_destroy: bool = False):
        self.explicitly_destroy = bool(explicitly_destroy)

    def _runtime_or_fail(self):
        if self.runtime is None:
            raise AssertionError('the buffer has been destroyed')
        return self.runtime

    @property
    def main_context(self):
        runtime = self.runtime
        return runtime.main_context if runtime is not None else None

    def print_memory_usage(self) -> None:
        self._runtime_or_fail().print_memory_usage()

    @abc.abstractmethod
    def destroy(self) -> None:
        """Only buffers built with `explicitly_destroy=True` may be destroyed by hand."""
        if not self.explicitly_destroy:
            raise AssertionError('explicitly_destroy=True is required to call destroy()')
        runtime, self.runtime = self.runtime, None
        if runtime is not None:
            runtime.destroy()
