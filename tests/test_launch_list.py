"""Launch lists without a GPU: who records what (the entry points here are stand-ins)."""

import ctypes
import threading

from burn_transformers_amd.kernels import library as K


class _FakeModule:
    """Stands where a kernel library stands: entry points that count their calls."""

    def __init__(self):
        self.launched = []

    def bt_fake_call(self, stream, call):
        self.launched.append(threading.get_ident())
        return 0


def test_a_list_records_the_calls_of_its_own_thread_only(monkeypatch):
    monkeypatch.setattr(K, "_held_stream", [0])          # no GPU here: any stream will do for a stand-in
    module, call = _FakeModule(), ctypes.c_int(0)
    program = K.Program()
    inside, may_go_on = threading.Event(), threading.Event()
    other_thread = []

    def other():
        inside.wait(5)
        K._launch(module, "bt_fake_call", call)        # another engine's step, say, while the list is open
        other_thread.append(threading.get_ident())
        may_go_on.set()

    worker = threading.Thread(target=other)
    worker.start()
    with program.recording():
        K._launch(module, "bt_fake_call", call)
        inside.set()
        assert may_go_on.wait(5)
        K._launch(module, "bt_fake_call", call)
    worker.join()
    assert len(program) == 2                           # the recording thread's two calls, kept and not launched
    assert module.launched == other_thread             # the other thread's call ran at once and was not kept
    K._launch(module, "bt_fake_call", call)            # after the recording: launched again
    assert len(program) == 2 and len(module.launched) == 2


def test_recording_while_launching_keeps_and_launches(monkeypatch):
    monkeypatch.setattr(K, "_held_stream", [0])
    module, call = _FakeModule(), ctypes.c_int(0)
    program = K.Program()
    with program.recording(launch=True):
        K._launch(module, "bt_fake_call", call)
    assert len(program) == 1 and len(module.launched) == 1
