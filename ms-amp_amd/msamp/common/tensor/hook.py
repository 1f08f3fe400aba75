"""Callback registry used for gradient post-hooks (msamp/common/tensor/hook.py:9-82)."""


class HookManager:
    """Ordered set of callbacks with the forward-hook signature fn(owner, inputs, output).

    Calling the manager with a value x calls fn(manager, (x,), x) for every registered fn, which is
    what a pass-through module's forward hooks would see.
    """
    class _RemoveHandle:
        def __init__(self, manager, hook_id):
            self.manager = manager
            self.hook_id = hook_id

        def remove(self):
            self.manager.hooks.pop(self.hook_id, None)

    def __init__(self):
        self.hooks = {}
        self.history_counter = 0

    def __call__(self, *args, **kwargs):
        output = args[0] if len(args) == 1 else args
        for fn in list(self.hooks.values()):
            fn(self, args, output)

    def register_hook(self, fn):
        """Register fn(owner, inputs, output) and return a handle whose remove() unregisters it."""
        hook_id = self.history_counter
        self.history_counter += 1
        self.hooks[hook_id] = fn
        return self._RemoveHandle(self, hook_id)
