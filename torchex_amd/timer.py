"""``TorchTimer``: wall-clock timing of GPU work between device synchronisations.

Same interface and printed line as the reference's timing helper
(``torchex/operator_py/timer.py:4-41``): ``timer.timing(name)`` returns a context
manager that synchronises the device on entry and exit, accumulates the elapsed
wall time and prints the running mean in milliseconds every ``print_freq``
uses; ``print_freq == -1`` switches a timer off.
"""
import time

import torch


class _NamedTimer:
    def __init__(self, name, print_freq):
        self.name = name
        self.print_freq = print_freq
        self.time_cost = 0.0
        self.begin_time = 0.0
        self.exe_counter = 0

    def reset(self):
        self.time_cost = 0.0
        self.exe_counter = 0

    @staticmethod
    def _sync():
        if torch.cuda.is_available():
            torch.cuda.synchronize()

    def __enter__(self):
        if self.print_freq > 0:
            self._sync()
            self.begin_time = time.time()
        return self

    def __exit__(self, exc_type, exc_val, exc_tb):
        if self.print_freq == -1:
            return
        self._sync()
        self.time_cost += time.time() - self.begin_time
        self.exe_counter += 1
        if self.exe_counter % self.print_freq == 0:
            print('Average time cost of {}: {:.4}ms'.format(
                self.name, self.time_cost / self.exe_counter * 1000))
            self.reset()


class TorchTimer:
    NamedTimer = _NamedTimer

    def __init__(self, print_freq=10):
        self.timer_dict = {}
        self.print_freq = print_freq

    def timing(self, name, freq=None):
        print_freq = freq if freq is not None else self.print_freq
        if name not in self.timer_dict:
            self.timer_dict[name] = _NamedTimer(name, print_freq)
        return self.timer_dict[name]
