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


class ContractError(RuntimeError):
    pass


KV_DTYPES = {"fp16", "bf16", "bf16-latent", "fp32", "fp4-e2m1-ue8m0-block32",
             "fp4-e2m1-ue8m0-block32-key-outlier1", "q4-bfp16-block32-key-outlier1",
             "q4-bfp16-block32", "q4-f16-per-head", "q5-q4-bfp16-block32",
             "fp8-e4m3-per-head"}
PREFILL_MODES = {"causal_blocked_exact", "causal_chunked", "causal_layer_major",
                 "causal_sequential"}


class ServiceView:
    """What the service's worker client makes of a ready line, and when it
    turns the worker down: the reading and the checks of CudaWorker.__init__
    (ops/python/expert_server.py:575-790), restated so that the worker's ready
    line can be held to them without the service.  `launch` carries the
    client's constructor arguments by name (max_context, requested_capacity,
    ram_cache_gib, vram_cache_gib, kv_page_tokens, placement_profile and the
    optional ones)."""

    def __init__(self, ready, launch):
        get = ready.get
        if get("type") != "ready":
            raise ContractError("worker did not become ready")
        self.protocol = int(get("protocol", 1))
        self.capacity = int(get("capacity", 1))
        self.architecture_id = str(get("architecture_id", ""))
        self.vocab_size = int(get("vocab_size", 0))
        self.model_max_context_tokens = int(get("max_context_tokens", 0))
        self.routed_layers = int(get("routed_layers", 0))
        self.experts_per_layer = int(get("experts_per_layer", 0))
        self.route_width = int(get("route_width", 0))
        self.expert_encoding = str(get("expert_encoding", ""))
        capabilities = get("operation_capabilities", [])
        self.operation_capabilities = list(capabilities) if isinstance(capabilities, list) else []
        self.prefill_mode = str(get("prefill_mode", ""))
        self.prefill_chunk_tokens = int(get("prefill_chunk_tokens", 0))
        self.session_retention = bool(get("session_retention", False))
        self.session_parking = bool(get("session_parking", False))
        self.session_persistence = bool(get("session_persistence", False))
        self.session_park_ram_bytes = int(get("session_park_ram_bytes", 0))
        self.session_park_page_capacity = int(get("session_park_page_capacity", 0))
        self.request_stream_mode = str(get("request_stream_mode", "default"))
        self.gpu_phase_timing = bool(get("gpu_phase_timing", False))
        self.sampling_supported = bool(get("sampling_supported", False))
        self.sampling_presence_penalty_supported = bool(
            get("sampling_presence_penalty_supported", False))
        self.mtp_resource_available = bool(get("mtp_resource_available", False))
        self.mtp_runtime_ready = bool(get("mtp_runtime_ready", False))
        self.mtp_enabled = bool(get("mtp_enabled", False))
        wanted_depth = launch.get("mtp_draft_depth")
        depth = get("mtp_draft_depth")
        if ((wanted_depth is not None and self.protocol < 13) or
                (self.protocol >= 13 and (isinstance(depth, bool) or
                                          not isinstance(depth, int) or depth < 0)) or
                (wanted_depth is not None and depth != wanted_depth)):
            raise ContractError("worker did not confirm the MTP execution policy")
        self.mtp_draft_depth = depth if self.protocol >= 13 else None
        self.retain_previous_route = bool(get("retain_previous_route", True))
        self.cpu_hybrid_enabled = bool(get("cpu_hybrid_enabled", False))
        if self.mtp_runtime_ready and not self.mtp_resource_available:
            raise ContractError("MTP runtime cannot be ready without resources")
        wanted = launch.get("retain_previous_route")
        if wanted is not None and self.retain_previous_route != wanted:
            raise ContractError("retained-route mode does not match the request")
        wanted = launch.get("enable_cpu_hybrid")
        if wanted is not None and self.cpu_hybrid_enabled != wanted:
            raise ContractError("CPU-hybrid mode does not match the request")
        self.rope_mode = str(get("rope_mode", "per_step_upload"))
        self.kv_dtype = str(get("kv_dtype", ""))
        self.kv_allocation = str(get("kv_allocation", ""))
        self.kv_page_tokens = int(get("kv_page_tokens", 0))
        self.kv_page_bytes = int(get("kv_page_bytes", 0))
        self.kv_page_capacity = int(get("kv_page_capacity", 0))
        self.placement_profile = str(get("placement_profile", ""))
        self.placement_mode = str(get("placement_mode", "budgeted"))
        self.ram_cache_bytes = int(get("ram_cache_bytes", 0))
        self.vram_cache_bytes = int(get("vram_cache_bytes", 0))
        self.routed_vram_policy = str(get("routed_vram_policy", "fixed"))
        self.placement_prefetch_enabled = bool(get("placement_prefetch_enabled", False))
        state = get("placement_prefetch_state")
        if state is None:      # protocol-4 workers published the boolean only
            state = "ready" if self.placement_prefetch_enabled else "disabled"
        self.placement_prefetch_state = str(state)
        self.placement_minimum_observations = int(get("placement_minimum_observations", 0))

        profile = launch["placement_profile"]
        policy = launch.get("routed_vram_policy", "fixed")
        ram_ceiling = launch["ram_cache_gib"] << 30
        budgeted_invalid = self.placement_mode == "budgeted" and (
            self.placement_profile != profile or
            not 0 < self.ram_cache_bytes <= ram_ceiling or
            not 0 < self.vram_cache_bytes or
            (policy == "fixed" and self.vram_cache_bytes > launch["vram_cache_gib"] << 30) or
            self.routed_vram_policy != policy or
            self.placement_prefetch_state not in {"disabled", "observing", "ready"} or
            self.placement_prefetch_enabled != (self.placement_prefetch_state == "ready") or
            (profile == "capacity" and self.placement_prefetch_state != "disabled") or
            self.placement_minimum_observations != (1 if profile == "latency" else 2))
        resident_invalid = self.placement_mode == "resident" and (
            self.placement_profile != "resident" or self.ram_cache_bytes != 0 or
            self.vram_cache_bytes <= 0 or self.placement_prefetch_enabled or
            self.placement_prefetch_state != "disabled" or
            self.placement_minimum_observations != 0)
        placement_invalid = (budgeted_invalid or resident_invalid or
                             self.placement_mode not in {"budgeted", "resident"} or
                             (self.protocol >= 11 and
                              self.routed_vram_policy not in {"fixed", "fit"}))
        routed = (self.routed_layers != 0 or self.experts_per_layer != 0 or
                  self.route_width != 0 or bool(self.expert_encoding))
        routed_invalid = routed and (
            self.routed_layers <= 0 or self.experts_per_layer <= 0 or
            not 1 <= self.route_width <= self.experts_per_layer or
            not self.expert_encoding)
        capabilities = self.operation_capabilities
        descriptor_invalid = self.protocol >= 6 and (
            not self.architecture_id or self.vocab_size <= 0 or
            self.model_max_context_tokens < launch["max_context"] or routed_invalid or
            not capabilities or len(set(capabilities)) != len(capabilities) or
            any(not isinstance(item, str) or not item for item in capabilities))
        parking_invalid = self.protocol >= 9 and (
            (self.session_parking and (
                not self.session_retention or
                not 0 < self.session_park_ram_bytes <= ram_ceiling or
                self.session_park_page_capacity <= 0)) or
            (not self.session_parking and (
                self.session_park_ram_bytes != 0 or self.session_park_page_capacity != 0)))
        persistence_invalid = self.protocol >= 12 and self.session_persistence and (
            not self.session_retention or not self.session_parking)
        sampling_invalid = self.protocol >= 10 and (
            self.sampling_presence_penalty_supported != self.sampling_supported)
        chunk_ceiling = launch.get("prefill_chunk_tokens", 0)
        if (self.protocol < 4 or descriptor_invalid or sampling_invalid or
                parking_invalid or persistence_invalid or
                self.capacity != launch["requested_capacity"] or
                self.prefill_mode not in PREFILL_MODES or
                not 1 <= self.prefill_chunk_tokens <= launch["max_context"] or
                (chunk_ceiling and self.prefill_chunk_tokens > chunk_ceiling) or
                self.kv_dtype not in KV_DTYPES or
                self.kv_allocation not in {"paged_on_demand", "preallocated"} or
                self.kv_page_tokens != launch["kv_page_tokens"] or
                self.kv_page_bytes <= 0 or self.kv_page_capacity <= 0 or
                placement_invalid):
            raise ContractError("worker does not support requested runtime contract")

    def sampling_fields(self, temperature, top_p, top_k, min_p, presence_penalty, seed):
        """The SAMPLING group the client appends to BEGIN
        (_sampling_command, expert_server.py:948-975)."""
        if not self.sampling_supported:
            return []
        fields = ["SAMPLING", round(temperature * 1_000_000), round(top_p * 1_000_000),
                  top_k, round(min_p * 1_000_000)]
        if self.sampling_presence_penalty_supported:
            fields.append(round(presence_penalty * 1_000_000))
        return fields + [seed]
