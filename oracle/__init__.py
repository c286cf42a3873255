"""TEST INFRASTRUCTURE: CPU oracle for the KV-cache hot path (checker only, never shipped)."""
