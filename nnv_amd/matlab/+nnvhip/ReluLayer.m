classdef ReluLayer < ReluLayer
    % ReluLayer whose relax-star reach (ReluLayer.m:72-150 -> PosLin.reach, PosLin.m:863-1650) runs on
    % the device.  The override sits at layer level because PosLin.multipleStepReachStarApprox_at_one
    % reads I.V directly (PosLin.m:702) and would force a device -> host fetch.
    methods
        function obj = ReluLayer(varargin)
            obj = obj@ReluLayer(varargin{:});
        end
        function images = reach_star_multipleInputs(obj, in_images, method, option, relaxFactor, dis_opt, lp_solver) %#ok<INUSL>
            % 'reduceMem' suffix (ReluLayer.m:107-112): split off for ImageStars only; for a Star the whole string
            % reaches PosLin.reach, which does not know it (PosLin.m:2165-2166)
            reduceMem = false;
            if contains(method, "reduceMem")
                for i = 1:length(in_images)
                    if ~isa(in_images(i), 'ImageStar')
                        error("This reachability method does not exist");
                    end
                end
                parts = split(string(method), '-');
                method = strjoin(parts(1:end-1), '-');
                reduceMem = true;
            end
            switch char(method)
                case 'relax-star-range', order = 2;                       % PosLin.m:934-936
                case 'relax-star-area',  order = 1;                       % PosLin.m:1049-1052
                case {'relax-star-bound', 'relax-star-ub', 'relax-star-random', 'relax-star-static'}
                    order = 0;                                            % ascending neuron index
                otherwise
                    error("This reachability method does not exist");
            end
            if relaxFactor < 0 || relaxFactor > 1
                error('Invalid relax factor');
            end
            n = length(in_images);
            hs = zeros(1, n, 'uint64');
            for i = 1:n, hs(i) = in_images(i).dev.h; end
            if relaxFactor == 1
                out = nnvhip_mex('relu_relax', order, relaxFactor, hs);
            else    % some bounds come from LPs first (host lpsolver fed from the resident set)
                out = zeros(1, n, 'uint64');
                for i = 1:n, out(i) = nnvhip.relaxed_star_lp(hs(i), method, relaxFactor, lp_solver, dis_opt); end
            end
            for i = n:-1:1
                if isa(in_images(i), 'ImageStar') && reduceMem
                    % ReluLayer.m:119-146: the box-like ImageStar of the estimated ranges, filled on the device
                    hh = in_images(i).height; ww = in_images(i).width; cc = in_images(i).numChannel;
                    [boxed, l, u] = nnvhip_mex('relu_reduce_mem', out(i), hh, ww, cc);
                    nnvhip_mex('star_release', out(i));
                    images(i) = nnvhip.ImageStar(nnvhip.DeviceSet(boxed), hh, ww, cc);
                    images(i).im_lb = reshape(l, hh, ww, cc);
                    images(i).im_ub = reshape(u, hh, ww, cc);
                elseif isa(in_images(i), 'ImageStar')
                    images(i) = nnvhip.ImageStar(nnvhip.DeviceSet(out(i)), in_images(i).height, in_images(i).width, in_images(i).numChannel);
                else
                    images(i) = nnvhip.Star(nnvhip.DeviceSet(out(i)));
                end
                if strcmp(dis_opt, 'display')
                    [idx, ~, ~, ninact] = nnvhip_mex('fetch_crossing', out(i));
                    fprintf('\n%d neurons with ub <= 0 are found by estimating ranges', ninact);
                    fprintf('\nConstruct new star set, %d new predicate variables are introduced', numel(idx));
                end
            end
        end
        function images = reach_star_single_input(obj, in_image, method, relaxFactor, dis_opt, lp_solver)
            images = obj.reach_star_multipleInputs(in_image, method, 'single', relaxFactor, dis_opt, lp_solver);
        end
    end
end
