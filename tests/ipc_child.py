"""Child process of the IPC export test: reopens tensors from the arguments `reduce_tensor` produced in the parent
(the payload the reference's sidecar client sends, sidecar/serde.py:89-95) and returns their bytes.  Started with the
`spawn` method, so nothing has touched the GPU in this process before the handles are opened."""

import sys


def main(conn) -> None:
    try:
        import torch   # noqa: F401  (first GPU use in this process happens inside the rebuild functions)

        payload = conn.recv()
        out = []
        for fn, args in payload:
            t = fn(*args)                   # opens the IPC memory handle
            out.append(t.cpu().view(torch.uint8).numpy().tobytes())
            del t
        conn.send(("ok", out))
    except Exception as e:  # the parent reports it
        conn.send(("error", f"{type(e).__name__}: {e}"))
    finally:
        conn.close()


if __name__ == "__main__":
    sys.exit(0)
