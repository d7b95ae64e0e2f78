"""Helpers shared by the benchmark definitions."""


def reset_workspace(C, workspace):
    """Untimed reset before every call: outputs and own flags cleared, preamble marked as done."""

    def reset():
        C.zero_()
        for buf in (workspace.locks, workspace.aux_buffer):
            if buf is not None:
                buf.zero_()
        workspace.prepared = True

    return reset
