"""CPU oracle for one Bamboo pipeline stage (TEST INFRASTRUCTURE ONLY).

Nothing in this package is part of the product.  It restates, in plain
Python / PyTorch-CPU, the algorithm of the reference path so that the HIP
implementation under ``bamboo_amd`` has something independent to be checked
against.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import it; ``bamboo_amd`` never does.

Modules
  schedule  instruction streams (1F1B TrainSchedule, eager-RC merge, next-stage,
            previous-stage and data-parallel failover merges)
            -- follows deepspeed/runtime/pipe/schedule.py
  layers    transformer layer / bottleneck block maths on torch CPU ops
            -- follows DeepSpeedExamples/pipeline_parallelism/{transformer,resnet}.py
  adam      the fused-Adam update formula -- follows csrc/adam/multi_tensor_adam.cu
  wire      flat wire format of whole layers with their Adam moments
            -- follows deepspeed/runtime/pipe/engine.py send_layers / recv_layers
  stage     interpreter that runs an instruction stream over the oracle layers
            with torch.autograd -- follows deepspeed/runtime/pipe/engine.py _exec_*

Pin status (what each function was checked against, see tests/test_oracle_*.py):
  schedule.step_to_micro_batch   closed form vs. the piecewise parity rules;
                                 brute-force invariants over S<=6, M<=10
  schedule.train_schedule        invariants of the upstream DeepSpeed unit test
                                 (tests/unit/test_pipe_schedule.py:126-157) and the
                                 hand trace S=4, M=4, stage 1
  schedule.eager_merge           hand trace + "RC F(k) directly before RecvGrad(k)"
  schedule.next_stage_failover   semantic pin: gradients of the merged stream equal
                                 those of own+shadow run as one stage
  schedule.prev_stage_failover   what its definition fixes: before curr_step only the
                                 own SendGrad of steps < failed_step, each once, then the
                                 own stream unchanged; end to end: a pipeline that loses
                                 a stage mid-batch ends with the gradients and weights of
                                 the run in which nothing fails (tests/test_gpu_pipeline.py)
  schedule.allreduce_failover    its definition (empty before failed_step, own after)
  wire.pack_layers/unpack_layers hand-written known answer with distinct elements (order of
                                 layers, parameters and moments), round trip
  layers.*                       reduce to torch library routines (linear, softmax,
                                 conv2d, batch_norm); custom LayerNorm checked against
                                 the closed form with torch.std (unbiased)
  adam.adam_step                 torch.optim.Adam / AdamW (fp32, <=2 ulp per step)
The reference publishes no stored tensors for this path, so tensor-level parity
against the reference's own run is "parity unpinned"; the checks above are what
the mathematics fixes.
"""
