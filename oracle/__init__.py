"""TEST INFRASTRUCTURE. CPU restatement of the reference's multi-adapter LoRA path, used only as the
checker by tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py. The product
(lorax_amd/) never imports it."""
