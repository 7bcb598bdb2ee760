"""Base class of the training-loop callbacks (``recis.hooks.hook``, hook.py:4-100): every method
is a no-op that a subclass overrides; the loop calls them at the points their names say."""


class Hook:
    def before_train(self, *args, **kwargs):
        pass

    def after_train(self, *args, **kwargs):
        pass

    def before_evaluate(self, *args, **kwargs):
        pass

    def after_evaluate(self, *args, **kwargs):
        pass

    def before_epoch(self, *args, **kwargs):
        pass

    def after_epoch(self, *args, **kwargs):
        pass

    def before_step(self, *args, **kwargs):
        pass

    def after_step(self, *args, **kwargs):
        pass

    def end(self, *args, **kwargs):
        pass
