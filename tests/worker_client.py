"""Drives the worker process over its stdin / stdout line protocol, the way
the service's worker client does (ops/python/expert_server.py:489-640): one
command line out, one JSON line back."""
import json
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "quantum-llm_amd", "bin", "qllm-worker")


def launch_arguments(max_context=256, kv_page_tokens=64, capacity=1, **extra):
    options = {"max-context": max_context, "ram-cache-gib": 1, "vram-cache-gib": 1,
               "capacity": capacity, "kv-cache-mib": 64, "kv-page-tokens": kv_page_tokens,
               "placement-profile": "latency"}
    options.update({name.replace("_", "-"): value for name, value in extra.items()})
    return [f"--{name}" if value is True else f"--{name}={value}"
            for name, value in options.items() if value is not None]


def run_to_exit(arguments, timeout=60):
    """For launches that are expected to fail before the ready line."""
    done = subprocess.run([BINARY, *arguments], stdin=subprocess.DEVNULL,
                          capture_output=True, text=True, timeout=timeout)
    return done.returncode, done.stdout, done.stderr


class Worker:
    def __init__(self, artifact, **options):
        self.process = subprocess.Popen(
            [BINARY, artifact, "--worker", *launch_arguments(**options)],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=subprocess.PIPE,
            text=True, bufsize=1)
        line = self.process.stdout.readline()
        if not line:
            raise RuntimeError("worker ended before ready: " + self.process.stderr.read())
        self.ready = json.loads(line)

    def send(self, *fields):
        self.process.stdin.write("\t".join(str(field) for field in fields) + "\n")
        self.process.stdin.flush()

    def ask(self, *fields):
        self.send(*fields)
        line = self.process.stdout.readline()
        if not line:
            raise RuntimeError("worker ended: " + self.process.stderr.read())
        return json.loads(line)

    def begin(self, request, context, tokens, sampling=None):
        fields = ["BEGIN", request, context, ",".join(str(int(t)) for t in tokens)]
        if sampling is not None:
            fields += ["SAMPLING", *sampling]
        return self.ask(*fields)

    def next(self, request, mode=0):
        return self.ask("NEXT", request, mode)

    def close(self):
        if self.process.poll() is None:
            self.process.stdin.close()
            self.process.wait(timeout=30)
        return self.process.returncode
