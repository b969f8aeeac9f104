"""Serving workloads: synthetic requests, a runner that feeds them to an engine, and the report."""

from .report import BenchReport, BenchRun, RequestTiming, format_report, percentile, report_json, summarize  # noqa: F401
from .runner import run_workload  # noqa: F401
from .workload import BenchRequest, assign_arrivals, parse_range, read_requests_jsonl, synthetic_requests  # noqa: F401
