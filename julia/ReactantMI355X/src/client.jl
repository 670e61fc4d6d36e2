# The "rocm" backend: a PJRT client made by libreactant_mi355x.so.
#
# Reference: src/accelerators/GPU.jl:7-37 (make_pjrt_client), :82-89 (registration under "rocm"
# when Reactant_jll was built for rocm), src/accelerators/Registration.jl:24-54 (register_backend),
# src/xla/XLA.jl:126-150 (`client("gpu")` tries "cuda", "metal", "rocm" in turn),
# src/xla/XLA.jl:228-233 (REACTANT_VISIBLE_GPU_DEVICES -> global_state.local_gpu_device_ids, which
# initialize_default_clients! passes on as `allowed_devices`, XLA.jl:300-303).

function make_pjrt_client(;
    node_id::Integer=0,
    num_nodes::Integer=1,
    distributed_runtime_client=nothing,
    allowed_devices::Union{Nothing,Vector{Int}}=nothing,
)
    num_nodes == 1 || error("ReactantMI355X runs on one process and one GPU (num_nodes = $num_nodes)")
    distributed_runtime_client === nothing ||
        error("ReactantMI355X has no distributed runtime (collectives are out of scope)")
    errstr = Ref{Cstring}(C_NULL)
    ids = allowed_devices === nothing ? Int64[] : Int64.(allowed_devices)
    GC.@preserve errstr ids begin
        client = ccall(
            sym(:MakeGPUClient),
            Ptr{Cvoid},
            (Cint, Cint, Ptr{Int64}, Int64, Cdouble, Bool, Cstring, Ptr{Cstring}, Ptr{Cvoid}),
            node_id,
            num_nodes,
            isempty(ids) ? Ptr{Int64}(C_NULL) : pointer(ids),
            length(ids),
            XLA.XLA_REACTANT_GPU_MEM_FRACTION[],   # honoured: the allocator's bytes_limit
            XLA.XLA_REACTANT_GPU_PREALLOCATE[],    # accepted; the caching allocator grows on demand
            "rocm",
            errstr,
            C_NULL,
        )
    end
    if client == C_NULL
        msg = errstr[] == C_NULL ? "MakeGPUClient failed" : XLA.unsafe_string_and_free(errstr[])
        throw(AssertionError(msg))
    end
    return PJRT.Client(client)
end

function register!()
    registered = any(b -> b.platform_name == "rocm", Reactant.Accelerators.Registration.RegisteredBackends)
    if registered
        @warn "ReactantMI355X: a \"rocm\" backend is already registered (Reactant_jll built for rocm); " *
              "not registering a second one.  Make the client by hand: ReactantMI355X.make_pjrt_client()"
        return nothing
    end
    Reactant.Accelerators.Registration.register_backend(
        "rocm"; priority=500, pjrt_initialize_function=make_pjrt_client
    )
    return nothing
end

# `XLA.device_properties` asks libReactantExtra for CUDA devices only and warns for everything else
# (src/xla/Device.jl:42-60); the compile pipeline formats a chip string from the result
# (src/compiler/Compiler.jl, target "rocm").  For devices of this library: a filled-in struct, no warning.
function mi355x_device_properties(device::PJRT.Device)
    props = Ref{API.DeviceProperties}()
    GC.@preserve props begin
        Base.Libc.memset(Base.unsafe_convert(Ptr{Cvoid}, props), 0, sizeof(API.DeviceProperties))
    end
    return props[]
end

function install_device_properties!()
    Core.eval(
        XLA,
        quote
            function device_properties(device::PJRT.Device)
                if $(owns)(device.device)
                    key = (Int(get_local_hardware_id(device)), "rocm")
                    return get!(() -> $(mi355x_device_properties)(device), DEVICE_PROPERTIES_CACHE, key)
                end
                return invoke(device_properties, Tuple{AbstractDevice}, device)
            end
        end,
    )
    return nothing
end
