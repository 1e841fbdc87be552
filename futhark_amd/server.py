"""Client for the line protocol of futhark_amd/bin/segops-server
(docs/server-protocol.rst of the reference): what `futhark bench` and
`futhark test` do on their side of the pipe."""
from __future__ import annotations

import subprocess
from pathlib import Path

SERVER = Path(__file__).resolve().parent / "bin" / "segops-server"


class ServerFailure(RuntimeError):
    """A command answered `%%% FAILURE`; the message is what followed."""


class Server:
    def __init__(self, *options: str):
        if not SERVER.exists():
            raise FileNotFoundError(f"{SERVER} is not built; run `python -m futhark_amd.build`")
        self.proc = subprocess.Popen([str(SERVER), *options], stdin=subprocess.PIPE,
                                     stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                                     bufsize=1)
        self._read_reply()  # the OK that ends initialisation

    def _read_reply(self) -> list[str]:
        lines, failed = [], None
        while True:
            line = self.proc.stdout.readline()
            if line == "":
                raise RuntimeError("server terminated: " + self.proc.stderr.read())
            line = line.rstrip("\n")
            if line == "%%% OK":
                break
            if line == "%%% FAILURE":
                failed = len(lines)
                continue
            lines.append(line)
        if failed is not None:
            raise ServerFailure("\n".join(lines[failed:]))
        return lines

    def cmd(self, *words) -> list[str]:
        def quote(w) -> str:
            w = str(w)
            return f'"{w}"' if (" " in w or w == "") else w
        self.proc.stdin.write(" ".join(quote(w) for w in words) + "\n")
        self.proc.stdin.flush()
        return self._read_reply()

    def call(self, entry: str, out: str, *ins: str) -> int:
        """Returns the runtime in microseconds the server reports."""
        for line in self.cmd("call", entry, out, *ins):
            if line.startswith("runtime: "):
                return int(line.split()[1])
        raise RuntimeError("no runtime line")

    def close(self) -> int:
        self.proc.stdin.close()
        return self.proc.wait(timeout=60)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        if self.proc.poll() is None:
            self.close()
