"""Compile server: one JSON request per line on stdin, one JSON reply per line.

Kernels are compiled in this separate process whenever the calling process has
PyTorch loaded: PyTorch brings its own copies of the runtime-compilation
libraries, and once they are loaded a process-local compile would go through
them instead of the ROCm installation's compiler. Compiling out of process
keeps the generated code the same wherever the request comes from.

Request : {"src": str, "opts": [str], "arch": str, "cache_dir": str}
Reply   : "FTR-REPLY " + {"ok": true, "path": cache file} | {"ok": true, "b64": code object}
          | {"ok": false, "error": str}
The reply line carries a marker so that a stray line some library prints on
stdout is not mistaken for it; the code object travels inline when the cache
directory cannot be written.
"""
import base64
import json
import os
import sys


def main():
    from flextensor_amd import runtime as rt
    assert "torch" not in sys.modules
    out = sys.stdout
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        try:
            req = json.loads(line)
            if req.get("cache_dir"):
                rt.CACHE_DIR = req["cache_dir"]
            code = rt.compile_to_code(req["src"], req["opts"], req.get("arch", rt.DEFAULT_ARCH),
                                      _in_process=True)
            path = os.path.join(rt.CACHE_DIR, rt.code_key(req["src"], req["opts"],
                                                          req.get("arch", rt.DEFAULT_ARCH)) + ".hsaco")
            if os.path.exists(path) and os.path.getsize(path) == len(code):
                rep = {"ok": True, "path": path}
            else:
                rep = {"ok": True, "b64": base64.b64encode(code).decode("ascii")}
        except Exception as e:  # noqa: BLE001
            rep = {"ok": False, "error": str(e)}
        out.write(rt.WORKER_REPLY_MARK + json.dumps(rep) + "\n")
        out.flush()


if __name__ == "__main__":
    main()
