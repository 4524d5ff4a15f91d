"""Compile server: one JSON request per line on stdin, one JSON reply per line.

Kernels are compiled in this separate process whenever the calling process has
PyTorch loaded: PyTorch brings its own copies of the runtime-compilation
libraries, and once they are loaded a process-local compile would go through
them instead of the ROCm installation's compiler. Compiling out of process
keeps the generated code the same wherever the request comes from.

Request : {"src": str, "opts": [str], "arch": str, "cache_dir": str}
Reply   : {"ok": true, "path": cache file} | {"ok": false, "error": str}
"""
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
            rt.compile_to_code(req["src"], req["opts"], req.get("arch", rt.DEFAULT_ARCH),
                               _in_process=True)
            path = os.path.join(rt.CACHE_DIR, rt.code_key(req["src"], req["opts"],
                                                          req.get("arch", rt.DEFAULT_ARCH)) + ".hsaco")
            rep = {"ok": True, "path": path}
        except Exception as e:  # noqa: BLE001
            rep = {"ok": False, "error": str(e)}
        out.write(json.dumps(rep) + "\n")
        out.flush()


if __name__ == "__main__":
    main()
